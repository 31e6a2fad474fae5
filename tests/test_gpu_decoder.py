"""The decoder glue ops and the Llama-shaped decoder stack on the device against CPU checkers.

RoPE has no counterpart in the reference repository, so it is checked against the closed form in float64; the
decoder as a whole is checked against tests/decoder_check.py (float64 numpy over oracle-dequantised weights).
Tolerances: fp32 paths (decode rows, prompts of at most 8 tokens) 1e-3 of the largest reference magnitude; the
bf16-operand MFMA prefill path 2e-2."""
import numpy as np
import pytest

from decoder_check import CheckDecoder
from gpu_util import dev

pytestmark = pytest.mark.gpu


def max_norm_err(got, ref):
    ref = np.asarray(ref, np.float64)
    return float(np.abs(np.asarray(got, np.float64) - ref).max() / max(np.abs(ref).max(), 1e-30))


def small_config():
    from skainet_amd.decoder import LlamaConfig
    return LlamaConfig(layers=2, hidden=512, heads=8, kv_heads=2, head_dim=64, ffn=1024, vocab=1024, ctx_max=64,
                       rope_theta=10000.0)


@pytest.fixture(scope="module")
def small_model(hip_backend):
    from skainet_amd.decoder import LlamaWeights
    cfg = small_config()
    w = LlamaWeights(cfg, seed=11, sigma=0.05, keep_host=True)
    return cfg, w


@pytest.mark.parametrize("tokens,heads,head_dim,pos0,pitch_extra", [(1, 8, 64, 0, 0), (5, 4, 128, 17, 0), (7, 2, 64, 3, 192)])
def test_rope_scatter_closed_form(hip_backend, torch_cuda, tokens, heads, head_dim, pos0, pitch_extra):
    torch = torch_cuda
    kx = hip_backend
    rng = np.random.default_rng(5)
    pitch = heads * head_dim + pitch_extra
    src = rng.standard_normal((tokens, pitch)).astype(np.float32)
    col0 = pitch_extra // 2
    theta = 500000.0
    x = src[:, col0:col0 + heads * head_dim].reshape(tokens, heads, head_dim).astype(np.float64)
    ang = (np.arange(tokens)[:, None, None] + pos0) * theta ** (-2.0 * np.arange(head_dim // 2)[None, None, :] / head_dim)
    want = np.empty_like(x)
    want[..., 0::2] = x[..., 0::2] * np.cos(ang) - x[..., 1::2] * np.sin(ang)
    want[..., 1::2] = x[..., 0::2] * np.sin(ang) + x[..., 1::2] * np.cos(ang)
    d_src = dev(torch, src)
    cap = 32
    # query layout: [heads, tokens, head_dim], rows from 0
    out_q = torch.zeros(heads * tokens * head_dim, dtype=torch.float32, device="cuda")
    kx.rope_scatter_dev(d_src.data_ptr() + 4 * col0, out_q, tokens, heads, head_dim, pos0, None, theta, True,
                        tokens * head_dim, False, in_row_pitch=pitch)
    # cache layout: [heads, cap, head_dim], rows at the absolute position, position read from the device
    out_c = torch.full((heads, cap, head_dim), 7.0, dtype=torch.float32, device="cuda")
    pos_dev = dev(torch, np.array([pos0], np.int32))
    kx.rope_scatter_dev(d_src.data_ptr() + 4 * col0, out_c, tokens, heads, head_dim, 0, pos_dev, theta, True,
                        cap * head_dim, True, in_row_pitch=pitch)
    # values: copied, not rotated
    out_v = torch.full((heads, cap, head_dim), 7.0, dtype=torch.float32, device="cuda")
    kx.rope_scatter_dev(d_src.data_ptr() + 4 * col0, out_v, tokens, heads, head_dim, pos0, None, theta, False,
                        cap * head_dim, True, in_row_pitch=pitch)
    kx.sync()
    got_q = out_q.cpu().numpy().reshape(heads, tokens, head_dim).transpose(1, 0, 2)
    assert np.abs(got_q - want).max() < 2e-5
    got_c = out_c.cpu().numpy()
    assert np.abs(got_c[:, pos0:pos0 + tokens].transpose(1, 0, 2) - want).max() < 2e-5
    untouched = np.ones(cap, bool)
    untouched[pos0:pos0 + tokens] = False
    assert (got_c[:, untouched] == 7.0).all()
    got_v = out_v.cpu().numpy()
    assert np.array_equal(got_v[:, pos0:pos0 + tokens].transpose(1, 0, 2), x.astype(np.float32))
    assert (got_v[:, untouched] == 7.0).all()


def test_rope_rejects_odd_head_dim(hip_backend, torch_cuda):
    from skainet_amd._lib import HipError
    t = torch_cuda.zeros(64, device="cuda")
    with pytest.raises(HipError):
        hip_backend.rope_scatter_dev(t, t, 1, 1, 7)


def test_heads_to_rows_and_swiglu_and_increment(hip_backend, torch_cuda):
    torch, kx = torch_cuda, hip_backend
    rng = np.random.default_rng(9)
    heads, tokens, hd = 6, 5, 32
    a = rng.standard_normal((heads, tokens, hd)).astype(np.float32)
    out = torch.empty(tokens * heads * hd, dtype=torch.float32, device="cuda")
    kx.heads_to_rows_dev(dev(torch, a), out, heads, tokens, hd)
    rows, ffn = 3, 130
    gu = (rng.standard_normal((rows, 2 * ffn)) * 3).astype(np.float32)
    act = torch.empty(rows * ffn, dtype=torch.float32, device="cuda")
    kx.swiglu_pairs_dev(dev(torch, gu), act, rows * ffn)
    ctr = dev(torch, np.array([41], np.int32))
    kx.i32_increment_dev(ctr, 1)
    kx.i32_increment_dev(ctr, 3)
    pos, klen = dev(torch, np.array([6], np.int32)), dev(torch, np.array([7], np.int32))
    tok, log = dev(torch, np.array([99], np.int32)), dev(torch, np.zeros(10, np.int32))
    kx.decode_advance_dev(pos, klen, tok, log, 9)
    kx.sync()
    assert int(pos.cpu()[0]) == 7 and int(klen.cpu()[0]) == 8 and log.cpu().tolist() == [0] * 7 + [99, 0, 0]
    # the position saturates at the capacity: two more steps fit (8, 9), the third changes nothing
    for _ in range(3):
        kx.decode_advance_dev(pos, klen, tok, log, 9)
    kx.sync()
    assert int(pos.cpu()[0]) == 9 and int(klen.cpu()[0]) == 9 and log.cpu().tolist() == [0] * 7 + [99, 99, 99]
    assert np.array_equal(out.cpu().numpy().reshape(tokens, heads, hd), a.transpose(1, 0, 2))
    g, u = gu[:, 0::2].astype(np.float64), gu[:, 1::2].astype(np.float64)
    assert max_norm_err(act.cpu().numpy().reshape(rows, ffn), g / (1 + np.exp(-g)) * u) < 1e-6
    assert int(ctr.cpu()[0]) == 45


def test_rope_qkv_equals_three_scatters(hip_backend, torch_cuda):
    torch, kx = torch_cuda, hip_backend
    rng = np.random.default_rng(31)
    tokens, heads, kvh, hd, cap, pos0, theta = 5, 8, 2, 64, 40, 9, 500000.0
    width = (heads + 2 * kvh) * hd
    qkv = dev(torch, rng.standard_normal((tokens, width)).astype(np.float32))
    pos_dev = dev(torch, np.array([pos0], np.int32))
    for use_dev_pos in (False, True):
        q1 = torch.zeros(heads * tokens * hd, device="cuda")
        k1 = torch.full((kvh * cap * hd,), 3.0, device="cuda")
        v1 = torch.full((kvh * cap * hd,), 3.0, device="cuda")
        q2, k2, v2 = torch.zeros_like(q1), torch.full_like(k1, 3.0), torch.full_like(v1, 3.0)
        pd = pos_dev if use_dev_pos else None
        ps = 0 if use_dev_pos else pos0
        kx.rope_qkv_dev(qkv, q1, k1, v1, tokens, heads, kvh, hd, cap, ps, pd, theta)
        base = qkv.data_ptr()
        kx.rope_scatter_dev(base, q2, tokens, heads, hd, ps, pd, theta, True, tokens * hd, False, in_row_pitch=width)
        kx.rope_scatter_dev(base + 4 * heads * hd, k2, tokens, kvh, hd, ps, pd, theta, True, cap * hd, True, in_row_pitch=width)
        kx.rope_scatter_dev(base + 4 * (heads + kvh) * hd, v2, tokens, kvh, hd, ps, pd, theta, False, cap * hd, True,
                            in_row_pitch=width)
        kx.sync()
        for a, b in ((q1, q2), (k1, k2), (v1, v2)):
            assert np.array_equal(a.cpu().numpy(), b.cpu().numpy())
    from skainet_amd._lib import HipError
    with pytest.raises(HipError):
        kx.rope_qkv_dev(qkv, q1, k1, v1, tokens, heads, kvh, hd, cap, cap - 2, None, theta)   # rows past the cache


@pytest.mark.parametrize("enc,n,k,m", [("Q4_K", 1536, 1024, 1), ("Q4_K", 1030, 512, 2), ("Q4_K", 24, 4096 + 256, 1),
                                        ("Q4_K", 640, 512, 5), ("Q6_K", 512, 512, 1), ("Q4_K", 768, 1024, 24),
                                        ("Q4_K", 1030, 14336, 1), ("Q4_K", 26, 16640, 1), ("Q4_K", 4096, 12288, 1), ("Q4_K", 2050, 8448, 1),
                                        ("Q4_K", 300, 512, 40), ("Q6_K", 258, 1024, 33), ("Q8_0", 130, 2048, 64),
                                        ("Q4_K", 64, 5120, 300), ("Q8_0", 66, 96, 12), ("Q4_K", 1030, 4096, 1), ("Q4_K", 14000, 2048, 1),
                                        ("Q4_K", 50, 3072, 1), ("Q4_K", 6, 1024, 1)])
def test_matmul_fused_equals_composed(hip_backend, torch_cuda, enc, n, k, m):
    """Every prologue / epilogue combination against float64 arithmetic on the oracle-decoded weight; the decode
    shapes of Q4_K run the one-kernel route (also with K of several passes), the other cases the composed route of the
    same entry."""
    from oracle import lib as O
    torch, kx = torch_cuda, hip_backend
    rng = np.random.default_rng(n + k + m)
    packed = kx.quantize(enc, (rng.standard_normal((n, k)) * 0.05).astype(np.float32))
    wd = O.dequant(enc, packed).reshape(n, k).astype(np.float64)
    w = kx.DeviceWeight.upload(enc, packed, n, k)
    x = (rng.standard_normal((m, k)) * 2).astype(np.float32)
    gain = (1 + 0.2 * rng.standard_normal(k)).astype(np.float32)
    res = rng.standard_normal((m, n)).astype(np.float32)
    eps = 1e-5
    tol = 2e-2 if m > 8 else 1e-3
    xd = x.astype(np.float64)
    xn = xd / np.sqrt((xd * xd).mean(1, keepdims=True) + eps) * gain
    d_x, d_gain = dev(torch, x), dev(torch, gain)
    for use_gain in (False, True):
        p = (xn if use_gain else xd) @ wd.T
        for epi in (kx.EPI_NONE, kx.EPI_RESIDUAL, kx.EPI_SWIGLU):
            want = p if epi == kx.EPI_NONE else p + res if epi == kx.EPI_RESIDUAL else \
                p[:, 0::2] / (1 + np.exp(-p[:, 0::2])) * p[:, 1::2]
            out = dev(torch, res.copy()) if epi == kx.EPI_RESIDUAL else torch.full((m, want.shape[1]), 9.0, device="cuda")
            w.matmul_fused(d_x, m, out, gain=d_gain if use_gain else None, eps=eps,
                           residual=out if epi == kx.EPI_RESIDUAL else None, epilogue=epi)   # residual aliases the output
            kx.sync()
            assert max_norm_err(out.cpu().numpy(), want) < tol, (use_gain, epi)
    if m > 8 and k % 256 == 0:
        # the same through forced K splits: the epilogue then runs in the launch that sums the splits
        try:
            for ks in (2, 3):
                kx.set_tuning("gemm_ksplit", ks)
                for epi in (kx.EPI_RESIDUAL, kx.EPI_SWIGLU):
                    p = xn @ wd.T
                    want = p + res if epi == kx.EPI_RESIDUAL else p[:, 0::2] / (1 + np.exp(-p[:, 0::2])) * p[:, 1::2]
                    out = dev(torch, res.copy()) if epi == kx.EPI_RESIDUAL else torch.full((m, want.shape[1]), 9.0, device="cuda")
                    w.matmul_fused(d_x, m, out, gain=d_gain, eps=eps, residual=out if epi == kx.EPI_RESIDUAL else None, epilogue=epi)
                    kx.sync()
                    assert max_norm_err(out.cpu().numpy(), want) < tol, (ks, epi)
        finally:
            kx.set_tuning("gemm_ksplit", 0)
    from skainet_amd._lib import HipError
    with pytest.raises(HipError):
        w.matmul_fused(d_x, m, out, epilogue=kx.EPI_RESIDUAL)          # residual epilogue without a residual
    with pytest.raises(HipError):
        w.matmul_fused(d_x, m, out, epilogue=7)


@pytest.mark.parametrize("enc,hidden,ffn,m", [("Q4_K", 512, 768, 40), ("Q4_K", 1024, 2816, 130), ("Q4_K", 256, 512, 3), ("Q6_K", 512, 512, 33),
                                               ("Q8_0", 96, 160, 12), ("Q4_K", 4096, 14336, 64)])
def test_mlp_swiglu_equals_float64_and_the_two_fused_products(hip_backend, torch_cuda, enc, hidden, ffn, m):
    """The gated MLP block in one call against float64 arithmetic on the oracle-decoded weights (2e-2 of the largest output
    for prompt rows on the bf16 matrix cores, 1e-3 for up to 8 rows) and against the two fused products it replaces, with
    and without the norm and the residual (aliasing the output); Q4_K prompt rows run the fragment-order kernel for the
    down projection when it is forced, with the SwiGLU in its rounding pass and the residual in its store."""
    from oracle import lib as O
    torch, kx = torch_cuda, hip_backend
    rng = np.random.default_rng(hidden + ffn + m)
    pgu = kx.quantize(enc, (rng.standard_normal((2 * ffn, hidden)) * 0.05).astype(np.float32))
    pdn = kx.quantize(enc, (rng.standard_normal((hidden, ffn)) * 0.05).astype(np.float32))
    wgu_h = O.dequant(enc, pgu).reshape(2 * ffn, hidden).astype(np.float64)
    wdn_h = O.dequant(enc, pdn).reshape(hidden, ffn).astype(np.float64)
    wgu, wdn = kx.DeviceWeight.upload(enc, pgu, 2 * ffn, hidden), kx.DeviceWeight.upload(enc, pdn, hidden, ffn)
    x = (rng.standard_normal((m, hidden)) * 2).astype(np.float32)
    gain = (1 + 0.2 * rng.standard_normal(hidden)).astype(np.float32)
    res = rng.standard_normal((m, hidden)).astype(np.float32)
    eps = 1e-5
    tol = 2e-2 if m > 8 else 1e-3
    xd = x.astype(np.float64)
    xn = xd / np.sqrt((xd * xd).mean(1, keepdims=True) + eps) * gain
    d_x, d_gain = dev(torch, x), dev(torch, gain)
    act = torch.empty((m, ffn), device="cuda")
    for frag in ((1, 2) if enc == "Q4_K" and m > 8 else (1,)):
        try:
            kx.set_tuning("gemm_frag", frag)
            for use_gain in (False, True):
                p = (xn if use_gain else xd) @ wgu_h.T
                a = p[:, 0::2] / (1 + np.exp(-p[:, 0::2])) * p[:, 1::2]
                for use_res in (False, True):
                    want = a @ wdn_h.T + (res if use_res else 0.0)
                    out = dev(torch, res.copy()) if use_res else torch.full((m, hidden), 9.0, device="cuda")
                    wgu.mlp_swiglu(wdn, d_x, m, out, gain=d_gain if use_gain else None, eps=eps, residual=out if use_res else None)
                    kx.sync()
                    if frag == 2:
                        assert kx.last_kernel() == "q4k_gemm_frag_kernel"
                    got = out.cpu().numpy()
                    assert max_norm_err(got, want) < tol, (frag, use_gain, use_res)
                    two = dev(torch, res.copy()) if use_res else torch.full((m, hidden), 9.0, device="cuda")
                    wgu.matmul_fused(d_x, m, act, gain=d_gain if use_gain else None, eps=eps, epilogue=kx.EPI_SWIGLU)
                    wdn.matmul_fused(act, m, two, residual=two if use_res else None, epilogue=kx.EPI_RESIDUAL if use_res else kx.EPI_NONE)
                    kx.sync()
                    # the same operands rounded at the same places: only the order of fp32 sums may differ
                    assert max_norm_err(got, two.cpu().numpy().astype(np.float64)) < 1e-4, (frag, use_gain, use_res)
        finally:
            kx.set_tuning("gemm_frag", 1)
    from skainet_amd._lib import HipError
    with pytest.raises(HipError):
        wdn.mlp_swiglu(wdn, d_x, m, act)                               # not a (gate, up) weight for this down projection


@pytest.mark.parametrize("enc,heads,kvh,hd,k", [("Q4_K", 8, 2, 64, 512), ("Q4_K", 32, 8, 128, 4096), ("Q4_K", 3, 1, 64, 256),
                                                ("Q6_K", 4, 2, 64, 512), ("Q4_K", 5, 1, 64, 1024), ("Q4_K", 8, 4, 128, 2048)])
def test_matmul_qkv_rope_equals_product_then_rope(hip_backend, torch_cuda, enc, heads, kvh, hd, k):
    """The one-launch decode projection (norm + product + RoPE + cache append) against the separate entries, with and
    without the norm, at a device-side position; rows of the caches other than the position stay untouched."""
    torch, kx = torch_cuda, hip_backend
    rng = np.random.default_rng(heads * hd + k)
    n, cap, pos, theta, eps = (heads + 2 * kvh) * hd, 24, 13, 500000.0, 1e-5
    w = kx.DeviceWeight.upload(enc, kx.quantize(enc, (rng.standard_normal((n, k)) * 0.05).astype(np.float32)), n, k)
    x = dev(torch, rng.standard_normal(k).astype(np.float32))
    gain = dev(torch, (1 + 0.1 * rng.standard_normal(k)).astype(np.float32))
    pos_dev = dev(torch, np.array([pos], np.int32))
    for g in (None, gain):
        q1 = torch.zeros(heads * hd, device="cuda")
        k1 = torch.full((kvh * cap * hd,), 5.0, device="cuda")
        v1 = torch.full((kvh * cap * hd,), 5.0, device="cuda")
        q2, k2, v2 = torch.zeros_like(q1), torch.full_like(k1, 5.0), torch.full_like(v1, 5.0)
        w.matmul_qkv_rope(x, q1, k1, v1, heads, kvh, hd, cap, pos_dev, theta, gain=g, eps=eps)
        # the same call with the per-token rotation table: identical bits
        table = torch.empty(hd, device="cuda")
        kx.rope_table_dev(pos_dev, theta, hd, table)
        q3, k3, v3 = torch.zeros_like(q1), torch.full_like(k1, 5.0), torch.full_like(v1, 5.0)
        w.matmul_qkv_rope(x, q3, k3, v3, heads, kvh, hd, cap, pos_dev, theta, gain=g, eps=eps, rope_table=table)
        kx.sync()
        assert torch.equal(q1, q3) and torch.equal(k1, k3) and torch.equal(v1, v3)
        qkv = torch.empty(n, device="cuda")
        w.matmul_fused(x, 1, qkv, gain=g, eps=eps)
        kx.rope_qkv_dev(qkv, q2, k2, v2, 1, heads, kvh, hd, cap, 0, pos_dev, theta)
        kx.sync()
        for a, b in ((q1, q2), (k1, k2), (v1, v2)):
            a, b = a.cpu().numpy(), b.cpu().numpy()
            assert np.abs(a - b).max() <= 1e-5 * max(np.abs(b).max(), 1.0)
            assert np.array_equal(a == 5.0, b == 5.0)
    from skainet_amd._lib import HipError
    with pytest.raises(HipError):
        w.matmul_qkv_rope(x, q1, k1, v1, heads + 1, kvh, hd, cap, pos_dev, theta)     # head shape does not match the rows


def test_sdpa_cache_layout_matches_contiguous(hip_backend, torch_cuda):
    """K / V read in place from a cache with spare rows == the contiguous-operand kernel on the gathered rows."""
    torch, kx = torch_cuda, hip_backend
    rng = np.random.default_rng(21)
    b, h, hkv, sq, skv, cap, d = 2, 8, 2, 3, 37, 50, 64
    q = rng.standard_normal((b, h, sq, d)).astype(np.float32)
    kc = rng.standard_normal((b, hkv, cap, d)).astype(np.float32)
    vc = rng.standard_normal((b, hkv, cap, d)).astype(np.float32)
    lens = np.array([37, 20], np.int32)
    out_c = torch.empty(b * h * sq * d, dtype=torch.float32, device="cuda")
    out_p = torch.empty_like(out_c)
    kx.sdpa_cache_dev(dev(torch, q), dev(torch, kc), dev(torch, vc), out_c, b, h, hkv, sq, skv, cap, d, 0.125, True, 0, 0,
                      dev(torch, lens))
    kx.sdpa_dev(dev(torch, q), dev(torch, kc[:, :, :skv]), dev(torch, vc[:, :, :skv]), out_p, b, h, hkv, sq, skv, d, 0.125,
                True, 0, 0, dev(torch, lens))
    kx.sync()
    assert np.array_equal(out_c.cpu().numpy(), out_p.cpu().numpy())
    from skainet_amd._lib import HipError
    with pytest.raises(HipError):
        kx.sdpa_cache_dev(out_c, out_c, out_c, out_p, 1, 8, 2, 1, 40, 39, 64, 1.0)


@pytest.mark.parametrize("b,h,hkv,sq,skv,cap,d", [(1, 32, 8, 512, 512, 2048, 128), (2, 8, 2, 40, 56, 64, 64), (2, 8, 2, 3, 37, 50, 64),
                                                    (1, 4, 4, 1, 9, 16, 32)])
def test_sdpa_cache_rows_is_the_head_major_result_transposed(hip_backend, torch_cuda, b, h, hkv, sq, skv, cap, d):
    """Attention with the output as token rows ([batch, seq_q, heads, head_dim]: the matrix-core prompt kernel stores it that
    way itself, other shapes go through a transposing pass) equals the head-major entry's result, element for element."""
    torch, kx = torch_cuda, hip_backend
    rng = np.random.default_rng(b + h + sq)
    q = dev(torch, rng.standard_normal((b, h, sq, d)).astype(np.float32))
    kc = dev(torch, rng.standard_normal((b, hkv, cap, d)).astype(np.float32))
    vc = dev(torch, rng.standard_normal((b, hkv, cap, d)).astype(np.float32))
    lens = dev(torch, np.array([skv, max(1, skv // 2)][:b], np.int32))
    heads_major = torch.full((b, h, sq, d), 7.0, device="cuda")
    rows = torch.full((b, sq, h, d), 9.0, device="cuda")
    scale = float(1.0 / np.sqrt(d))
    kx.sdpa_cache_dev(q, kc, vc, heads_major, b, h, hkv, sq, skv, cap, d, scale, True, 0, 0, lens)
    kx.sdpa_cache_rows_dev(q, kc, vc, rows, b, h, hkv, sq, skv, cap, d, scale, True, 0, 0, lens)
    kx.sync()
    assert np.array_equal(rows.cpu().numpy(), heads_major.cpu().numpy().transpose(0, 2, 1, 3))
    from skainet_amd._lib import HipError
    with pytest.raises(HipError):
        kx.sdpa_cache_rows_dev(q, kc, vc, rows, b, h, 3, sq, skv, cap, d, scale)        # heads not a multiple of kv_heads


def test_graph_replays_match_eager(hip_backend, torch_cuda):
    """A recorded sequence (norm -> packed GEMV -> add -> counter) replayed several times, with eager work and
    synchronisation between the replays, gives the eager result every time."""
    torch, kx = torch_cuda, hip_backend
    rng = np.random.default_rng(2)
    n, k = 768, 512
    w = kx.DeviceWeight.upload("Q4_K", kx.quantize("Q4_K", (rng.standard_normal((n, k)) * 0.05).astype(np.float32)), n, k)
    gain = dev(torch, np.ones(k, np.float32))
    x = dev(torch, rng.standard_normal(k).astype(np.float32))
    xn = torch.empty(k, dtype=torch.float32, device="cuda")
    y = torch.empty(n, dtype=torch.float32, device="cuda")
    acc = torch.zeros(n, dtype=torch.float32, device="cuda")
    ctr = dev(torch, np.zeros(1, np.int32))

    def step():
        kx.rms_norm_dev(x, gain, xn, 1, k, 1e-5)
        w.matmul(xn, 1, y)
        kx.add_dev(acc, y, acc, n)
        kx.i32_increment_dev(ctr, 1)

    step()
    kx.sync()
    y1 = y.cpu().numpy().copy()
    with kx.Graph() as g:
        step()
    kx.sync()
    assert int(ctr.cpu()[0]) == 1, "recording must not execute the step"
    for i in range(4):
        g.launch()
        g.sync()
        kx.rms_norm_dev(x, gain, xn, 1, k, 1e-5)      # eager work between replays
        kx.sync()
        assert int(ctr.cpu()[0]) == 2 + i
        assert np.array_equal(y.cpu().numpy(), y1)
        assert max_norm_err(acc.cpu().numpy(), y1.astype(np.float64) * (2 + i)) < 1e-6
    g.close()


def test_graph_is_refused_once_scratch_moved(hip_backend, torch_cuda):
    """A recorded graph holds the scratch addresses of its recording. When a later call makes the library reallocate
    that scratch, launching the graph is refused on the host (nothing runs, a message says why); a call that would grow
    scratch inside an open capture fails instead of freeing memory under the capture."""
    import threading
    torch, kx = torch_cuda, hip_backend
    from skainet_amd import _lib
    result = {}

    def worker():                                   # a fresh thread: its scratch starts empty, whatever ran before
        try:
            heads, kvh, d = 8, 2, 64
            q = torch.randn((1, heads, 1, d), device="cuda")
            out = torch.empty_like(q)

            def attend(skv):                        # single-query attention: split-key partials live in the workspace
                k = torch.randn((1, kvh, skv, d), device="cuda")
                v = torch.randn((1, kvh, skv, d), device="cuda")
                kx.sdpa_dev(q, k, v, out, 1, heads, kvh, 1, skv, d, 0.125, False)
                return k, v

            keep = attend(512)                      # sizes the workspace (1 MiB granule)
            kx.sync()
            # a prompt-shaped product parks 4 MiB of bf16 activations in the same workspace
            from gpu_util import random_valid_blocks
            n, kk, m = 1024, 4096, 512
            wbig = kx.DeviceWeight.upload("Q4_K", random_valid_blocks("Q4_K", n * kk // 256, 5), n, kk)
            xbig = torch.randn((m, kk), device="cuda")
            ybig = torch.empty((m, n), device="cuda")
            # growth inside a capture is refused
            assert _lib.hip().skainet_hip_graph_begin() == 0
            rc_inside = _lib.hip().skainet_hip_matmul_dev(wbig._h, xbig.data_ptr(), m, ybig.data_ptr())
            msg_inside = _lib.last_error()
            g_aborted = _lib.hip().skainet_hip_graph_end()
            if g_aborted:
                _lib.hip().skainet_hip_graph_free(g_aborted)
            result["inside"] = (rc_inside, msg_inside)
            # a good recording, then the workspace grows: the graph is stale
            with kx.Graph() as g:
                kx.sdpa_dev(q, keep[0], keep[1], out, 1, heads, kvh, 1, 512, d, 0.125, False)
            g.launch(); g.sync()
            assert g.valid()
            wbig.matmul(xbig, m, ybig)
            kx.sync()
            result["valid_after"] = g.valid()
            try:
                g.launch()
                result["launch"] = "ran"
            except kx.HipError as e:
                result["launch"] = str(e)
            g.close()
            kx.thread_release()
        except Exception as e:                      # surfaces in the main thread's assert
            result["error"] = repr(e)

    t = threading.Thread(target=worker)
    t.start(); t.join()
    assert "error" not in result, result
    assert result["inside"][0] == -1 and "capture is open" in result["inside"][1], result
    assert result["valid_after"] is False
    assert "refused" in result["launch"] and "record it again" in result["launch"], result


def test_decoder_rerecords_its_graph_after_a_longer_prompt(small_model):
    """prefill(short) -> decode(graph) -> prefill(longer: the MFMA path grows the workspace) -> decode: the decoder
    notices the stale graph and records a new one; tokens equal the eager route's."""
    from skainet_amd.decoder import LlamaDecoder
    cfg, w = small_model
    rng = np.random.default_rng(21)
    short, longer = rng.integers(0, cfg.vocab, 3), rng.integers(0, cfg.vocab, 40)
    dec = LlamaDecoder(w, max_prefill=40)
    dec.prefill(short)
    dec.decode(3, use_graph=True)
    first = dec.prefill(longer)
    toks = dec.decode(5, use_graph=True)
    ref = LlamaDecoder(w, max_prefill=40)
    assert ref.prefill(longer) == first
    assert np.array_equal(ref.decode(5, use_graph=False), toks)
    dec.close(); ref.close()


def test_decode_stops_at_the_end_of_the_cache(small_model):
    """Replaying the recorded step past the context limit writes nothing: the position saturates, the cache rows and
    the token log keep their contents, and the host entry points refuse to go there in the first place."""
    from skainet_amd.decoder import LlamaDecoder
    cfg, w = small_model
    dec = LlamaDecoder(w, max_prefill=8)
    dec.prefill(np.arange(5) % cfg.vocab)
    with pytest.raises(ValueError):
        dec.decode_timed(cfg.ctx_max)               # 5 + 64 > 64
    dec.decode(cfg.ctx_max - 5, use_graph=True)     # exactly to the end
    assert dec.position() == cfg.ctx_max
    log_before = dec.generated.download(np.int32, cfg.ctx_max + 1)
    k_before = dec.k_cache.download(np.float32, cfg.layers * dec.kv_layer_floats)
    for _ in range(3):
        dec._graph.launch()                         # what a caller that skips the check would do
    dec._graph.sync()
    assert dec.position() == cfg.ctx_max
    assert np.array_equal(dec.generated.download(np.int32, cfg.ctx_max + 1), log_before)
    assert np.array_equal(dec.k_cache.download(np.float32, cfg.layers * dec.kv_layer_floats), k_before)
    dec.close()


def test_prefill_rejects_token_ids_outside_the_vocabulary(small_model):
    from skainet_amd.decoder import LlamaDecoder
    cfg, w = small_model
    dec = LlamaDecoder(w, max_prefill=4)
    for bad in ([0, cfg.vocab, 1], [3, -1], [2 ** 31 + 5]):
        with pytest.raises(ValueError, match="outside the vocabulary"):
            dec.prefill(np.array(bad, np.int64))
    dec.close()


def test_row_gather_clamps_ids_on_the_device(hip_backend, torch_cuda):
    """Ids that never pass through a host (a sampled token fed back) cannot read outside the weight: the gather clamps."""
    torch, kx = torch_cuda, hip_backend
    rows, cols = 16, 512
    packed = kx.quantize("Q4_K", (np.random.default_rng(4).standard_normal((rows, cols)) * 0.05).astype(np.float32))
    w = kx.DeviceWeight.upload("Q4_K", packed, rows, cols)
    dense = torch.empty(rows * cols, device="cuda")
    w.dequantize(dense)
    ids = dev(torch, np.array([3, -5, rows + 1000, rows - 1], np.int32))
    out = torch.empty(4 * cols, device="cuda")
    w.dequantize_rows(ids, 4, out)
    kx.sync()
    d, o = dense.cpu().numpy().reshape(rows, cols), out.cpu().numpy().reshape(4, cols)
    assert np.array_equal(o, d[[3, 0, rows - 1, rows - 1]])


@pytest.mark.parametrize("prompt_len,tol", [(6, 1e-3), (24, 2e-2)])
def test_prefill_matches_cpu_checker(small_model, prompt_len, tol):
    from skainet_amd.decoder import LlamaDecoder
    cfg, w = small_model
    prompt = np.random.default_rng(prompt_len).integers(0, cfg.vocab, prompt_len)
    dec = LlamaDecoder(w, max_prefill=32)
    tok = dec.prefill(prompt)
    chk = CheckDecoder(cfg, w.host)
    h_ref, logits_ref = chk.forward(prompt)
    assert max_norm_err(dec.hidden_rows(prompt_len), h_ref) < tol
    logits = dec.last_logits()
    assert max_norm_err(logits, logits_ref) < tol
    assert tok == int(np.argmax(logits)), "greedy token is the first arg-max of the device logits"
    assert dec.position() == prompt_len
    # the cache holds the rotated keys / raw values at rows [0, prompt_len) of every kv head
    for li in (0, cfg.layers - 1):
        kc = dec.k_cache.download(np.float32, dec.kv_layer_floats, 4 * li * dec.kv_layer_floats)
        vc = dec.v_cache.download(np.float32, dec.kv_layer_floats, 4 * li * dec.kv_layer_floats)
        kc = kc.reshape(cfg.kv_heads, cfg.ctx_max, cfg.head_dim)[:, :prompt_len]
        vc = vc.reshape(cfg.kv_heads, cfg.ctx_max, cfg.head_dim)[:, :prompt_len]
        assert max_norm_err(kc, chk.k[li]) < tol
        assert max_norm_err(vc, chk.v[li]) < tol


@pytest.mark.parametrize("use_graph", [False, True])
def test_greedy_decode_matches_cpu_checker(small_model, use_graph):
    """Teacher-forced on the device's own tokens: after every step the device logits match the checker's for the
    same token history, the emitted token is the first arg-max of the device logits, and it equals the checker's
    arg-max whenever the checker's top-2 gap is clear of the tolerance."""
    from skainet_amd.decoder import LlamaDecoder
    cfg, w = small_model
    prompt = np.random.default_rng(77).integers(0, cfg.vocab, 5)
    dec = LlamaDecoder(w, max_prefill=8)
    chk = CheckDecoder(cfg, w.host)
    tok = dec.prefill(prompt)
    _, logits_ref = chk.forward(prompt)
    steps = 12
    for i in range(steps):
        assert max_norm_err(dec.last_logits(), logits_ref) < 1e-3, f"step {i}"
        top2 = np.sort(logits_ref)[-2:]
        if top2[1] - top2[0] > 2e-3 * np.abs(logits_ref).max():
            assert tok == int(np.argmax(logits_ref)), f"step {i}"
        _, logits_ref = chk.forward([tok])
        nxt = int(dec.decode(1, use_graph=use_graph)[0])
        assert nxt == int(np.argmax(dec.last_logits()))
        assert dec.position() == len(prompt) + i + 1
        tok = nxt
    assert max_norm_err(dec.last_logits(), logits_ref) < 1e-3


def test_graph_and_eager_decode_agree(small_model):
    from skainet_amd.decoder import LlamaDecoder
    cfg, w = small_model
    prompt = np.random.default_rng(3).integers(0, cfg.vocab, 7)
    outs = []
    for use_graph in (False, True):
        dec = LlamaDecoder(w, max_prefill=8)
        first = dec.prefill(prompt)
        toks = dec.decode(10, use_graph=use_graph)
        assert np.array_equal(dec.generated_tokens(), np.concatenate([[first], toks]))   # the device-side token log
        outs.append((first, toks, dec.last_logits()))
    assert outs[0][0] == outs[1][0]
    assert np.array_equal(outs[0][1], outs[1][1])
    assert np.array_equal(outs[0][2], outs[1][2])


def test_decode_runs_with_the_one_row_matrix_core_kernel_switched_off(small_model):
    """A decode step's attention leaves its key splits unmerged for the output projection only where that projection's
    kernel will take them; with the kernel switched off the step falls back to attention + merge + product and gives
    the same tokens (fp32 row kernels: the checker's bound holds as before)."""
    from skainet_amd import kernels as kx
    from skainet_amd.decoder import LlamaDecoder
    cfg, w = small_model
    prompt = np.random.default_rng(5).integers(0, cfg.vocab, 6)
    ref = LlamaDecoder(w, max_prefill=8)
    first = ref.prefill(prompt)
    toks = ref.decode(6, use_graph=False)
    kx.set_tuning("q4k_mfma_enable", 0)
    try:
        dec = LlamaDecoder(w, max_prefill=8)
        assert dec.prefill(prompt) == first
        got = dec.decode(6, use_graph=False)
        assert max_norm_err(dec.last_logits(), ref.last_logits()) < 1e-3
    finally:
        kx.set_tuning("q4k_mfma_enable", 1)
    assert np.array_equal(got, toks)


def test_prefill_rejects_oversized_prompt(small_model):
    from skainet_amd.decoder import LlamaDecoder
    cfg, w = small_model
    dec = LlamaDecoder(w, max_prefill=4)
    with pytest.raises(ValueError):
        dec.prefill(np.zeros(5, np.int32))
    dec.prefill(np.zeros(4, np.int32))
    with pytest.raises(ValueError):
        dec.decode(cfg.ctx_max, use_graph=False)


def test_gguf_round_trip_gives_the_same_model(small_model, tmp_path):
    """Export the synthetic model as a llama-architecture GGUF file (separate q / k / v and gate / up tensors, llama.cpp
    names), load it back through the memory-mapped reader (which re-fuses them) and decode: same bytes on the device,
    so the tokens and logits are identical; a packed tensor uploaded straight from the mapping multiplies like the
    original."""
    from skainet_amd import gguf
    from skainet_amd.decoder import LlamaDecoder, LlamaWeights
    cfg, w = small_model
    path = str(tmp_path / "model.gguf")
    w.to_gguf(path)
    w2 = LlamaWeights.from_gguf(path, keep_host=True)
    from dataclasses import replace
    assert w2.cfg.rms_eps == pytest.approx(cfg.rms_eps, rel=1e-6)            # stored as float32 in the file
    assert replace(w2.cfg, rms_eps=cfg.rms_eps) == cfg
    for name, a in w.host.items():
        assert np.array_equal(np.asarray(a).reshape(-1), np.asarray(w2.host[name]).reshape(-1)), name
    prompt = np.random.default_rng(5).integers(0, cfg.vocab, 6)
    outs = []
    for weights in (w, w2):
        dec = LlamaDecoder(weights, max_prefill=8)
        first = dec.prefill(prompt)
        outs.append((first, dec.decode(6, use_graph=False), dec.last_logits()))
    assert outs[0][0] == outs[1][0] and np.array_equal(outs[0][1], outs[1][1]) and np.array_equal(outs[0][2], outs[1][2])
    with gguf.GGUFReader(path) as r:
        assert r.fields["llama.block_count"] == cfg.layers
        dw = r.upload("blk.1.ffn_down.weight")
        assert (dw.rows, dw.cols, dw.encoding) == (cfg.hidden, cfg.ffn, "Q4_K")
    from skainet_amd import kernels as kx
    import torch
    x = torch.randn(cfg.ffn, device="cuda")
    y1, y2 = torch.empty(cfg.hidden, device="cuda"), torch.empty(cfg.hidden, device="cuda")
    dw.matmul(x, 1, y1)
    w.layers[1].w_down.matmul(x, 1, y2)
    kx.sync()
    assert torch.equal(y1, y2)


@pytest.mark.parametrize("linear,head", [("Q5_K", "Q5_0"), ("Q4_0", "Q5_1")])
def test_decoder_over_the_other_packed_formats(hip_backend, linear, head, tmp_path):
    """The same stack with Q5_K / Q4_0 linears and Q5_0 / Q5_1 heads (composed launches: only Q4_K has the fused decode
    kernels; the 8-token prompt runs exact-fp32 row kernels): prefill and greedy decode against the float64 checker,
    and the model survives a GGUF round trip."""
    import dataclasses
    from skainet_amd.decoder import LlamaDecoder, LlamaWeights
    cfg = dataclasses.replace(small_config(), linear_encoding=linear, head_encoding=head)
    w = LlamaWeights(cfg, seed=13, sigma=0.05, keep_host=True)
    prompt = np.random.default_rng(3).integers(0, cfg.vocab, 8)
    dec = LlamaDecoder(w, max_prefill=32)
    tok = dec.prefill(prompt)
    chk = CheckDecoder(cfg, w.host)
    h_ref, logits_ref = chk.forward(prompt)
    assert max_norm_err(dec.hidden_rows(len(prompt)), h_ref) < 1e-3
    assert max_norm_err(dec.last_logits(), logits_ref) < 1e-3
    assert tok == int(np.argmax(dec.last_logits()))
    for i in range(4):
        _, logits_ref = chk.forward([tok])
        tok = int(dec.decode(1, use_graph=i > 0)[0])
        assert max_norm_err(dec.last_logits(), logits_ref) < 1e-3, f"step {i}"
        assert tok == int(np.argmax(dec.last_logits()))
    path = str(tmp_path / "m.gguf")
    w.to_gguf(path)
    w2 = LlamaWeights.from_gguf(path, ctx_max=cfg.ctx_max, keep_host=True)
    assert w2.cfg.linear_encoding == linear and w2.cfg.head_encoding == head
    for name, a in w.host.items():
        assert np.array_equal(np.asarray(a), np.asarray(w2.host[name])), name


# ---- the host-array route of the kernel SPI -------------------------------------------------------------------------
@pytest.mark.parametrize("enc,n,k", [("Q4_K", 1536, 1024), ("Q4_K", 260, 512), ("Q6_K", 130, 768), ("Q8_0", 96, 64)])
def test_host_array_product_equals_the_device_entry(hip_backend, torch_cuda, enc, n, k):
    """skainet_hip_matmul_host against skainet_hip_matmul_dev on the same handle, bit for bit: a large call, a smaller
    one on the re-used staging, then a batch that crosses into the GEMM path; padding around the host output stays."""
    from oracle import golden as G
    torch = torch_cuda
    blocks = G.weight_blocks(enc, n, k // G.PACKED[enc][0], 0xC0FFEE)
    w = hip_backend.DeviceWeight.upload(enc, G.row_major(blocks), n, k)
    for m in (5, 1, 12):
        a = G.floats(m * k, 0x1234 + m).reshape(m, k)
        padded = np.full(m * n + 8, 7, np.float32)
        out = padded[4:4 + m * n].reshape(m, n)
        w.matmul_host(a, out)
        want = torch.empty(m, n, device="cuda:0", dtype=torch.float32)
        w.matmul(dev(torch, a), m, want)
        torch.cuda.synchronize()
        assert np.array_equal(out.view(np.uint32), want.cpu().numpy().view(np.uint32)), f"m={m}"
        assert (padded[:4] == 7).all() and (padded[-4:] == 7).all()
    with pytest.raises(ValueError):
        w.matmul_host(np.zeros((2, k + 1), np.float32), np.zeros((2, n), np.float32))
    with pytest.raises(TypeError):
        w.matmul_host(np.zeros((2, k), np.float64), np.zeros((2, n), np.float32))
    w.matmul_host(np.zeros((0, k), np.float32), np.zeros((0, n), np.float32))      # nothing to do is not an error
    w.close()


def test_spi_route_decoder_follows_the_resident_decoder(small_model):
    """The decoder written against host arrays only (every linear through the host-array entry, attention and norms
    through the SPI's host kernels, the rest in numpy) produces the resident decoder's logits within the fp32 bar on a
    shared token history, and the checker's."""
    from skainet_amd.decoder import LlamaDecoder
    from skainet_amd.spi_decoder import SpiDecoder
    cfg, w = small_model
    prompt = np.random.default_rng(5).integers(0, cfg.vocab, 6)
    dec = LlamaDecoder(w, max_prefill=8)
    spi = SpiDecoder(w)
    chk = CheckDecoder(cfg, w.host)
    tok = dec.prefill(prompt)
    spi.prefill(prompt)
    _, logits_ref = chk.forward(prompt)
    for i in range(8):
        assert max_norm_err(spi.logits[0], logits_ref) < 1e-3, f"step {i}"
        assert max_norm_err(spi.logits[0], dec.last_logits()) < 1e-3, f"step {i}"
        assert spi.pos == dec.position()
        nxt = int(dec.decode(1, use_graph=False)[0])
        spi.step(tok)                      # teacher-forced on the resident decoder's token
        _, logits_ref = chk.forward([tok])
        tok = nxt
    per_token = 4 * cfg.layers + 1
    assert spi.matmul_calls == per_token * (len(prompt) + 8)
    with pytest.raises(ValueError):
        spi.step(cfg.vocab)
    spi.close()


# ---- attention + output projection as a pair (the projection merges the attention's key splits) ---------------------
@pytest.mark.parametrize("heads,kvh,hd,n,keys,bound,window,merged", [
    (32, 8, 128, 512, 576, 1024, 0, True),      # the Llama-3 head shape: 6 splits of 96 keys
    (32, 8, 128, 260, 1, 512, 0, True),         # one key
    (32, 8, 128, 512, 37, 64, 0, True),         # one split
    (32, 8, 128, 512, 1000, 1024, 256, True),   # sliding window inside the cache
    (16, 4, 64, 128, 200, 512, 0, True),        # 16 heads per K slice
    (4, 2, 256, 64, 130, 512, 0, True),         # 4 heads per K slice
    (32, 8, 128, 512, 1500, 2048, 0, False),    # more keys per split than the pair accepts: merge launch + product
    (8, 2, 64, 128, 100, 512, 0, False),        # 512 inputs: not a whole K slice
])
def test_attention_projection_pair_equals_its_parts(hip_backend, torch_cuda, heads, kvh, hd, n, keys, bound, window, merged):
    """skainet_hip_attn_out_proj_dev against attention into a buffer followed by the fused product, with and without a
    residual that aliases the output; the key count comes from the device, the bound from the host. Both routes
    accumulate in fp32 in different orders: 2e-5 of the largest output."""
    import oracle.golden as G
    torch, kx = torch_cuda, hip_backend
    rng = np.random.default_rng(heads * 1000 + keys)
    k = heads * hd
    cap = bound + 16
    blocks = G.weight_blocks("Q4_K", n, k // 256, 0xA77E)
    w = kx.DeviceWeight.upload("Q4_K", G.row_major(blocks), n, k)
    q = dev(torch, rng.standard_normal((heads, hd)).astype(np.float32))
    kc = dev(torch, rng.standard_normal((kvh, cap, hd)).astype(np.float32))
    vc = dev(torch, rng.standard_normal((kvh, cap, hd)).astype(np.float32))
    lens = dev(torch, np.array([keys], np.int32))
    res = rng.standard_normal(n).astype(np.float32)
    scale = float(1.0 / np.sqrt(hd))
    attn = torch.empty(k, dtype=torch.float32, device="cuda")
    tmp = torch.full((k,), float("nan"), dtype=torch.float32, device="cuda")
    for residual in (False, True):
        want = dev(torch, res.copy())
        kx.sdpa_cache_dev(q, kc, vc, attn, 1, heads, kvh, 1, bound, cap, hd, scale, True, window, 0, lens)
        w.matmul_fused(attn, 1, want, residual=want if residual else None, epilogue=kx.EPI_RESIDUAL if residual else kx.EPI_NONE)
        got = dev(torch, res.copy())
        w.attn_out_proj(q, kc, vc, heads, kvh, hd, bound, cap, scale, got, tmp, residual=got if residual else None,
                        window=window, lengths=lens)
        kx.sync()
        assert ("attention-merge" in kx.last_kernel()) == merged
        a, b = got.cpu().numpy(), want.cpu().numpy()
        assert np.isfinite(a).all()
        assert np.abs(a - b).max() <= 2e-5 * np.abs(b).max(), (residual, np.abs(a - b).max(), np.abs(b).max())
    # the switch takes the pair back to its parts, bit for bit
    kx.set_tuning("attn_merge_enable", 0)
    try:
        got = torch.empty(n, dtype=torch.float32, device="cuda")
        w.attn_out_proj(q, kc, vc, heads, kvh, hd, bound, cap, scale, got, tmp, lengths=lens, window=window)
        want = torch.empty(n, dtype=torch.float32, device="cuda")
        kx.sdpa_cache_dev(q, kc, vc, attn, 1, heads, kvh, 1, bound, cap, hd, scale, True, window, 0, lens)
        w.matmul_fused(attn, 1, want)
        kx.sync()
        assert "attention-merge" not in kx.last_kernel()
        assert np.array_equal(got.cpu().numpy(), want.cpu().numpy())
    finally:
        kx.set_tuning("attn_merge_enable", 1)
    from skainet_amd._lib import HipError
    with pytest.raises(HipError):
        w.attn_out_proj(q, kc, vc, heads + 1, kvh, hd, bound, cap, scale, got, tmp)
    w.close()


def test_decoder_crosses_a_key_bucket_with_its_graph(hip_backend):
    """The recorded step is laid out for a bound on the key count; when the cache outgrows it the decoder records
    again, and the tokens are the ones the eager route emits."""
    from skainet_amd.decoder import LlamaConfig, LlamaDecoder, LlamaWeights
    cfg = LlamaConfig(layers=2, hidden=1024, heads=8, kv_heads=2, head_dim=128, ffn=1024, vocab=512, ctx_max=96, rope_theta=10000.0)
    w = LlamaWeights(cfg, seed=5, sigma=0.05)
    prompt = np.random.default_rng(9).integers(0, cfg.vocab, 7)
    outs = []
    for use_graph in (False, True):
        dec = LlamaDecoder(w, max_prefill=8)
        dec.KEY_BUCKET = 16                      # buckets of 16 keys: the 40 steps cross two edges
        first = dec.prefill(prompt)
        toks = dec.decode(40, use_graph=use_graph)
        assert dec.position() == 47
        if use_graph:
            assert dec._graph_bound == 48
        outs.append((first, toks, dec.last_logits()))
        dec.close()
    assert outs[0][0] == outs[1][0]
    assert np.array_equal(outs[0][1], outs[1][1])
    assert np.array_equal(outs[0][2], outs[1][2])
