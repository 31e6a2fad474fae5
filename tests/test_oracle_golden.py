"""Pins the CPU oracle (oracle/skainet_oracle.c) before anything is compared against it.

Sources of truth, in order: the reference's own golden digests (tests/golden/reference_goldens.json, transcribed
from Goldens.kt), known answers of the reference's unit tests, the reference's C library compiled from its own
sources (oracle/_ref, when built) or the vectors recorded from it (tests/golden/ref_vectors.npz), and closed forms.
"""
import json
import os

import numpy as np
import pytest

from oracle import golden as G
from oracle import lib as L

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDENS = json.load(open(os.path.join(HERE, "golden", "reference_goldens.json")))
ENCS = ["Q8_0", "Q4_K", "Q6_K", "Q4_0", "Q5_0", "Q5_1", "Q5_K"]
NATIVE_ENCS = ["Q8_0", "Q4_K", "Q6_K"]          # the formats the reference's native C library covers


# ---- fp16 ----------------------------------------------------------------------------------------------
def test_half_to_float_matches_ieee_for_every_pattern():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    lib = L.oracle()
    got = np.array([lib.orc_half_to_float(int(b)) for b in bits], dtype=np.float32)
    finite = np.isfinite(want)
    assert np.array_equal(got[finite].view(np.uint32), want[finite].view(np.uint32))
    assert np.array_equal(np.isinf(got), np.isinf(want)) and np.array_equal(np.isnan(got), np.isnan(want))


def test_float_to_half_is_round_to_nearest_even():
    rng = np.random.default_rng(1)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001, 6.1e-5, 5.96e-8,
                  1.0009765625, 1.00048828125, 1.00146484375], dtype=np.float32)])
    lib = L.oracle()
    got = np.array([lib.orc_float_to_half(float(v)) for v in vals], dtype=np.uint16)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)


# ---- decode + exact GEMV: the reference's golden digests -------------------------------------------------
@pytest.mark.parametrize("enc", ENCS)
def test_decode_golden(enc):
    blocks = G.weight_blocks(enc, 4, 3, 0x5EED0001)   # PackedDecodeGoldenTest.kt:29-31
    assert G.digest(L.dequant(enc, G.row_major(blocks))) == GOLDENS[f"decode/{enc}"]


@pytest.mark.parametrize("enc", ENCS)
def test_transpose_golden(enc):
    bs = G.PACKED[enc][0]
    blocks = G.weight_blocks(enc, 4, 3, 0x5EED0003)   # PackedTransposeGoldenTest.kt:35-37
    dec = L.dequant(enc, G.row_major(blocks)).reshape(4, 3 * bs)
    assert G.digest(np.ascontiguousarray(dec.T)) == GOLDENS[f"transpose/{enc}"]
    # the block-major permutation decodes to the same matrix
    bm = L.dequant(enc, G.block_major(blocks)).reshape(3, 4, bs).transpose(1, 0, 2).reshape(4, 3 * bs)
    assert np.array_equal(bm.view(np.uint32), dec.view(np.uint32))


@pytest.mark.parametrize("enc", ENCS)
def test_scalar_matmul_golden(enc):
    bs = G.PACKED[enc][0]
    out_dim, nblocks, batch, seed = 4, 3, 3, 0x5EED0002   # ScalarKernelGoldenTest.kt:16-34
    blocks = G.weight_blocks(enc, out_dim, nblocks, seed)
    x = G.floats(batch * nblocks * bs, seed + 100).reshape(batch, nblocks * bs)
    y = L.gemv(enc, x, G.block_major(blocks), out_dim, row_major=False)
    assert G.digest(y) == GOLDENS[f"scalar-matmul/{enc}"]
    # canonical order through the row-major addressing: same bits (dispatch-bridge golden = first row)
    y_rm = L.gemv(enc, x, G.row_major(blocks), out_dim, row_major=True)
    assert np.array_equal(y.view(np.uint32), y_rm.view(np.uint32))
    assert G.digest(y_rm[0]) == GOLDENS[f"dispatch-bridge/{enc}"]


def test_relayout_is_the_tagged_block_permutation():
    # PackedLayoutFixtures (PackedLayoutFixtures.kt:44-106): 4 rows x 3 blocks, every block tagged with (row, block)
    rows, bpr, nb = 4, 3, 34
    canon = np.zeros((rows, bpr, nb), np.uint8)
    for o in range(rows):
        for b in range(bpr):
            canon[o, b, :] = 16 * o + b
    out = np.empty(canon.size, np.uint8)
    L.oracle().orc_relayout(L.u8(canon.reshape(-1)), L.u8(out), rows, bpr, nb, 0)
    assert np.array_equal(out.reshape(bpr, rows, nb)[:, :, 0], (16 * np.arange(rows)[None, :] + np.arange(bpr)[:, None]))
    back = np.empty_like(out)
    L.oracle().orc_relayout(L.u8(out), L.u8(back), rows, bpr, nb, 1)
    assert np.array_equal(back, canon.reshape(-1))


# ---- Q8_0 quantizer: known answers of Q8_0QuantizerTest.kt ----------------------------------------------
def _q8(values):
    v = np.ascontiguousarray(values, np.float32)
    out = np.empty(v.size // 32 * 34, np.uint8)
    L.oracle().orc_q8_0_quantize(L.fp(v), v.size, L.u8(out))
    return out


def test_q8_0_quantizer_known_answers():
    v = ((np.arange(32) - 16) * np.float32(0.1)).astype(np.float32)
    v[5] = 2.54
    b = _q8(v)                                                          # Q8_0QuantizerTest.kt:24-34
    d = b[:2].view(np.float16)[0]
    assert abs(float(d) - 2.54 / 127) < 1e-5
    assert b[2 + 5].view(np.int8) == 127
    assert b[2 + 0].view(np.int8) == int(np.round(np.float32(-1.6) / (np.float32(2.54) / np.float32(127))))
    assert not _q8(np.zeros(32, np.float32)).any()                      # :59-63
    # scale byte pattern = IEEE RNE of amax/127
    rng = np.random.default_rng(3)
    w = rng.standard_normal(32 * 64).astype(np.float32)
    q = _q8(w).reshape(-1, 34)
    want_d = (np.abs(w.reshape(-1, 32)).max(1) / np.float32(127)).astype(np.float16)
    assert np.array_equal(q[:, :2].copy().view(np.float16).ravel(), want_d)
    # round trip within half a code step (:36-57)
    back = L.dequant("Q8_0", q.reshape(-1)).reshape(-1, 32)
    amax = np.abs(w.reshape(-1, 32)).max(1, keepdims=True)
    assert (np.abs(back - w.reshape(-1, 32)) <= amax / 127 * 0.5 + 1e-3 * amax).all()


# ---- fused rows: closed forms and the reference C library ------------------------------------------------
def fill(size, seed, scale=1.0):
    """NativeFusedKernelsTest.kt:49"""
    i = np.arange(size, dtype=np.int64)
    return ((((i * 31 + seed * 17) % 23) - 11) / np.float32(11.0) * np.float32(scale)).astype(np.float32)


def test_rms_norm_matches_fp64_closed_form():
    rows, cols = 5, 96
    x, g = fill(rows * cols, 1), fill(cols, 2)
    out = np.empty_like(x)
    L.oracle().orc_f32_rms_norm(L.fp(x), L.fp(g), L.fp(out), rows, cols, 1e-6)
    xd = x.reshape(rows, cols).astype(np.float64)
    want = xd / np.sqrt((xd * xd).mean(1, keepdims=True) + 1e-6) * g.astype(np.float64)
    np.testing.assert_allclose(out.reshape(rows, cols), want, rtol=1e-4, atol=1e-4)   # NativeFusedKernelsTest.kt:122-132


def sdpa_fp64(q, k, v, scale, causal, window, rc, lengths, mask):
    """Textbook attention in float64 with the dense additive form of the rules (AttentionMask.additive)."""
    b, h, sq, d = q.shape
    hkv, skv = k.shape[1], k.shape[2]
    rep = h // hkv
    kk, vv = np.repeat(k, rep, 1).astype(np.float64), np.repeat(v, rep, 1).astype(np.float64)
    s = np.einsum("bhqd,bhkd->bhqk", q.astype(np.float64), kk) * scale
    qi, ki = np.arange(sq)[:, None], np.arange(skv)[None, :]
    absq = skv - sq + qi
    for bi in range(b):
        ok = np.ones((sq, skv), bool)
        if causal:
            ok &= ki <= absq
        if window > 0:
            ok &= (ki >= absq - window + 1) & (ki <= absq + rc)
        if lengths is not None:
            ok &= ki < lengths[bi]
        s[bi][:, ~ok] = -1e30
    if mask is not None:
        m = mask.reshape((1,) * (4 - mask.ndim) + mask.shape).astype(np.float64)
        if m.shape[1] == hkv and hkv != h:
            m = np.repeat(m, rep, 1)
        s = s + m
    s = s - s.max(-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(-1, keepdims=True)
    return np.einsum("bhqk,bhkd->bhqd", p, vv)


SDPA_GRID = [(h, hkv, sq, skv, causal, lengths, win, rc)
             for (h, hkv) in [(4, 4), (4, 2)] for (sq, skv) in [(6, 6), (3, 10), (1, 7)] for causal in (False, True)
             for lengths in (False, True) for (win, rc) in [(0, 0), (3, 0), (4, 2)]]   # NativeFusedKernelsTest.kt:169-183


def sdpa_inputs(batch, heads, kv_heads, sq, skv, d, seed=0):
    return (fill(batch * heads * sq * d, 1 + seed).reshape(batch, heads, sq, d),
            fill(batch * kv_heads * skv * d, 2 + seed).reshape(batch, kv_heads, skv, d),
            fill(batch * kv_heads * skv * d, 3 + seed).reshape(batch, kv_heads, skv, d))


@pytest.mark.parametrize("case", SDPA_GRID)
def test_sdpa_oracle_every_rule(case):
    h, hkv, sq, skv, causal, use_len, win, rc = case
    batch, d = 3, 8
    q, k, v = sdpa_inputs(batch, h, hkv, sq, skv, d)
    lengths = np.array([skv, (skv + 1) // 2, 1], np.int32) if use_len else None
    scale = 1.0 / np.sqrt(d)
    got = L.sdpa(q, k, v, scale, causal, win, rc, lengths)
    want = sdpa_fp64(q, k, v, scale, causal, win, rc, lengths, None)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5)
    if L.ref() is not None:
        np.testing.assert_allclose(got, L.sdpa(q, k, v, scale, causal, win, rc, lengths, lib=L.ref()), rtol=1e-4, atol=1e-5)


def test_sdpa_oracle_masks_padding_and_gqa():
    q, k, v = sdpa_inputs(2, 4, 2, 5, 9, 16, seed=4)
    for mask in (fill(9, 6).reshape(1, 1, 1, 9), fill(45, 7).reshape(5, 9), fill(2 * 4 * 5 * 9, 8).reshape(2, 4, 5, 9),
                 fill(2 * 2 * 5 * 9, 9).reshape(2, 2, 5, 9)):
        got = L.sdpa(q, k, v, 0.3, True, mask=mask)
        np.testing.assert_allclose(got, sdpa_fp64(q, k, v, 0.3, True, 0, 0, None, mask), rtol=1e-4, atol=1e-5)
        if L.ref() is not None:
            np.testing.assert_allclose(got, L.sdpa(q, k, v, 0.3, True, mask=mask, lib=L.ref()), rtol=1e-4, atol=1e-5)
    # fully padded row: finite and uniform over all keys (NativeFusedKernelsTest.kt:203-209)
    q, k, v = sdpa_inputs(2, 2, 2, 3, 5, 4)
    out = L.sdpa(q, k, v, 0.5, lengths=np.array([0, 5], np.int32))
    assert np.isfinite(out).all()
    np.testing.assert_allclose(out[0], np.broadcast_to(v[0].mean(1, keepdims=True), out[0].shape), rtol=1e-5, atol=1e-6)
    # GQA == MHA over tiled K/V (SdpaGqaParityTest.kt:19); decode == last row of prefill
    q, k, v = sdpa_inputs(1, 8, 2, 6, 6, 16, seed=2)
    a = L.sdpa(q, k, v, 0.25, True)
    b = L.sdpa(q, np.repeat(k, 4, 1), np.repeat(v, 4, 1), 0.25, True)
    assert np.array_equal(a, b)
    last = L.sdpa(np.ascontiguousarray(q[:, :, -1:, :]), k, v, 0.25, True)
    np.testing.assert_allclose(last, a[:, :, -1:, :], rtol=1e-6, atol=1e-7)


def test_softmax_and_dense_matmuls_against_numpy():
    x = fill(7 * 33, 5).reshape(7, 33) * 3
    out = np.empty_like(x)
    L.oracle().orc_f32_softmax_rows(L.fp(x), L.fp(out), 7, 33, 0)
    e = np.exp(x.astype(np.float64) - x.max(1, keepdims=True))
    np.testing.assert_allclose(out, e / e.sum(1, keepdims=True), rtol=1e-5, atol=1e-7)
    L.oracle().orc_f32_softmax_rows(L.fp(x), L.fp(out), 7, 33, 1)
    np.testing.assert_allclose(out, x - (np.log(e.sum(1, keepdims=True)) + x.max(1, keepdims=True)), rtol=1e-5, atol=1e-5)
    a, b = fill(5 * 12, 1).reshape(5, 12), fill(9 * 7, 2).reshape(9, 7)
    c = np.full((5, 8), 7.0, np.float32)
    L.oracle().orc_fp32_matmul(L.fp(a), 1, 12, L.fp(b), 0, 7, L.fp(c), 1, 8, 4, 7, 9)   # offsets and strides exercised
    aa = np.lib.stride_tricks.as_strided(a.reshape(-1)[1:], (4, 9), (48, 4))
    np.testing.assert_allclose(np.lib.stride_tricks.as_strided(c.reshape(-1)[1:], (4, 7), (32, 4)), aa.astype(np.float64) @ b, rtol=1e-5, atol=1e-6)
    assert c[0, 0] == 7.0
    w = fill(6 * 9, 3).reshape(6, 9)
    o = np.empty((4, 6), np.float32)
    L.oracle().orc_fp32_matmul_wt(L.fp(np.ascontiguousarray(aa)), 0, L.fp(w), 0, L.fp(o), 0, 4, 6, 9)
    np.testing.assert_allclose(o, aa.astype(np.float64) @ w.T, rtol=1e-5, atol=1e-6)


# ---- the int8-activation port against the reference-built library -----------------------------------------
@pytest.mark.parametrize("enc", NATIVE_ENCS)
def test_native_port_is_bit_identical_to_the_reference_library(enc):
    ref = L.ref()
    vec_path = os.path.join(HERE, "golden", "ref_vectors.npz")
    bs = G.PACKED[enc][0]
    n, nblocks = 6, 3
    blocks = G.weight_blocks(enc, n, nblocks, 0x5EED0010)
    w = G.row_major(blocks)
    x = G.floats(nblocks * bs, 0x5EED0011)
    short = {"Q8_0": "q8_0", "Q4_K": "q4k", "Q6_K": "q6k"}[enc]
    y = np.empty(n, np.float32)
    getattr(L.oracle(), f"orc_native_{short}_matmul_rm")(L.fp(x), 0, L.u8(w), 0, nblocks * bs, n, L.fp(y), 0)
    recorded = np.load(vec_path)[f"native_rm/{enc}"]
    if enc == "Q8_0":   # the reference compiles this float loop with -ffast-math: order may differ at ULP scale
        np.testing.assert_allclose(y, recorded, rtol=1e-5, atol=1e-5)
    else:               # integer dots: exact
        assert np.array_equal(y.view(np.uint32), recorded.view(np.uint32))
    if ref is not None:
        yr = np.empty(n, np.float32)
        getattr(ref, f"skainet_{short}_matmul_rm")(L.fp(x), 0, L.u8(w), 0, nblocks * bs, n, L.fp(yr), 0)
        assert np.array_equal(yr.view(np.uint32), recorded.view(np.uint32))
        # feed-order entry of the reference == its row-major entry (RowMajorMatmulParityTest.kt:25)
        yb = np.empty(n, np.float32)
        getattr(ref, f"skainet_{short}_matmul")(L.fp(x), 0, L.u8(G.block_major(blocks)), 0, nblocks * bs, n, L.fp(yb), 0)
        np.testing.assert_allclose(yb, yr, rtol=1e-6, atol=1e-6)
    # and the int8 path stays within the documented 3 % RMS of the exact kernel (NativeQ4KMatmulKernelParityTest.kt:84-103)
    exact = L.gemv(enc, x, w, n)
    assert np.sqrt(((y - exact) ** 2).mean()) / np.sqrt((exact ** 2).mean()) < 0.03


@pytest.mark.parametrize("enc", ["Q4_0", "Q5_0", "Q5_1", "Q5_K"])
def test_exact_kernels_of_the_other_formats_against_the_reference_library(enc):
    """The reference's C kernels for these formats multiply in fp32 (no int8 activations); they and the oracle's
    restatement of the Kotlin scalar kernels differ by summation order only."""
    bs = G.PACKED[enc][0]
    n, nblocks = 6, 3
    blocks = G.weight_blocks(enc, n, nblocks, 0x5EED0010)
    w = G.row_major(blocks)
    x = G.floats(nblocks * bs, 0x5EED0011)
    recorded = np.load(os.path.join(HERE, "golden", "ref_vectors.npz"))[f"native_rm/{enc}"]
    got = L.gemv(enc, x, w, n)
    scale = np.abs(recorded).max()
    assert np.abs(got - recorded).max() <= 1e-5 * scale
    ref = L.ref()
    if ref is not None and getattr(ref, f"skainet_{L._SHORT[enc]}_matmul_rm", None) is not None:
        yr, yb = np.empty(n, np.float32), np.empty(n, np.float32)
        getattr(ref, f"skainet_{L._SHORT[enc]}_matmul_rm")(L.fp(x), 0, L.u8(w), 0, nblocks * bs, n, L.fp(yr), 0)
        assert np.array_equal(yr.view(np.uint32), recorded.view(np.uint32))
        getattr(ref, f"skainet_{L._SHORT[enc]}_matmul")(L.fp(x), 0, L.u8(G.block_major(blocks)), 0, nblocks * bs, n, L.fp(yb), 0)
        np.testing.assert_allclose(yb, yr, rtol=1e-6, atol=1e-6 * scale)


def narrow_inputs(kind):
    """A (5 x 37, fp32) and B (37 x 11) as bf16 / fp16 bytes: seeded, with the specials of the format in B's first row
    (zero, negative zero, the smallest subnormal, the largest finite value)."""
    m, n, k = 5, 11, 37
    a = G.floats(m * k, 0x5EED0020).reshape(m, k)
    b = G.floats(k * n, 0x5EED0021).reshape(k, n) * 3
    if kind == "bf16":
        bits = (b.view(np.uint32) >> 16).astype("<u2")
        bits[0, :4] = [0x0000, 0x8000, 0x0001, 0x7F7F]
    else:
        bits = b.astype("<f2").view("<u2").copy()
        bits[0, :4] = [0x0000, 0x8000, 0x0001, 0x7BFF]
    return a, np.ascontiguousarray(bits).view(np.uint8).reshape(-1), m, n, k


def narrow_values(kind, b_bytes, k, n):
    bits = b_bytes.view("<u2").reshape(k, n)
    return (bits.astype(np.uint32) << 16).view(np.float32) if kind == "bf16" else bits.view("<f2").astype(np.float32)


@pytest.mark.parametrize("kind", ["bf16", "fp16"])
def test_narrow_float_matmul(kind):
    """ScalarBf16MatmulKernel.kt:19-46 (and the fp16 twin): numpy's own decode of the 16-bit values, float64 sums; the
    reference C library's result (recorded, and live when built); byte offset / strides; k == 0 zeroes the block;
    integer-valued operands give exact sums whatever the order."""
    a, b, m, n, k = narrow_inputs(kind)
    got = L.narrow_matmul(kind, a, b, m, n, k)
    bv = narrow_values(kind, b, k, n)
    want = a.astype(np.float64) @ bv.astype(np.float64)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5 * np.abs(want).max())
    recorded = np.load(os.path.join(HERE, "golden", "ref_vectors.npz"))[f"narrow/{kind}"]
    np.testing.assert_allclose(got, recorded, rtol=1e-5, atol=1e-5 * np.abs(want).max())
    if L.ref() is not None and getattr(L.ref(), f"skainet_{kind}_matmul", None) is not None:
        assert np.array_equal(L.narrow_matmul(kind, a, b, m, n, k, lib=L.ref()).view(np.uint32), recorded.view(np.uint32))
    # offsets and strides: a sub-block of A (rows 1.., columns 2..), of B (rows 2.., columns 3..) into a wider C
    fn = getattr(L.oracle(), f"orc_{kind}_matmul")
    c = np.full((m, 16), 7.0, np.float32)
    mm, nn, kk = m - 1, n - 3, k - 2
    fn(L.fp(a), 1 * k + 2, k, L.u8(b), 2 * n * 2 + 3 * 2, 2 * n, L.fp(c), 16 + 1, 16, mm, nn, kk)
    sub = a[1:, 2:].astype(np.float64) @ bv[2:, 3:].astype(np.float64)
    np.testing.assert_allclose(c[1:, 1:1 + nn], sub, rtol=1e-5, atol=1e-5 * np.abs(sub).max())
    assert (c[0] == 7.0).all() and (c[:, 0] == 7.0).all() and (c[:, 1 + nn:] == 7.0).all()
    fn(L.fp(a), 0, k, L.u8(b), 0, 2 * n, L.fp(c), 0, 16, m, n, 0)
    assert (c[:, :n] == 0.0).all() and (c[:, n:] == 7.0).all()
    # small integers: every product and partial sum is representable, so the result is exact
    rng = np.random.default_rng(3)
    ai = rng.integers(-8, 9, (m, k)).astype(np.float32)
    bi = rng.integers(-8, 9, (k, n)).astype(np.float32)
    bb = (bi.view(np.uint32) >> 16).astype("<u2") if kind == "bf16" else bi.astype("<f2").view("<u2")
    exact = L.narrow_matmul(kind, ai, np.ascontiguousarray(bb).view(np.uint8).reshape(-1), m, n, k)
    assert np.array_equal(exact, ai @ bi)


def test_recorded_reference_sdpa_vectors():
    """Vectors written by tests/golden/make_ref_vectors.py from the reference C library pin the oracle's attention."""
    z = np.load(os.path.join(HERE, "golden", "ref_vectors.npz"))
    for i, case in enumerate(SDPA_GRID):
        h, hkv, sq, skv, causal, use_len, win, rc = case
        q, k, v = sdpa_inputs(3, h, hkv, sq, skv, 8)
        lengths = np.array([skv, (skv + 1) // 2, 1], np.int32) if use_len else None
        got = L.sdpa(q, k, v, 1.0 / np.sqrt(8), causal, win, rc, lengths)
        np.testing.assert_allclose(got, z[f"sdpa/{i}"], rtol=1e-4, atol=1e-5)
