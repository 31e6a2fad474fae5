"""Host-side GGUF quantizers (skainet_amd/csrc/ggml_quant.c).

Q8_0 has a reference implementation (Q8_0Quantizer.kt) and is checked byte-for-byte against the oracle's
restatement of it; Q4_0 has one too (Q4_0Quantizer.kt) and is held to the known answers of the reference's own
Q4_0QuantizerTest.kt. Q4_K / Q6_K / Q5_K / Q5_0 / Q5_1 have none in the reference (parity unpinned): they are pinned
through the bit-exact decoder by invariants -- valid blocks, round trip within one code step, determinism, idempotence.
"""
import numpy as np
import pytest

from oracle import lib as L
from skainet_amd import kernels


def weights(rows, cols, seed=0, sigma=0.02):
    return (np.random.default_rng(seed).standard_normal((rows, cols)) * sigma).astype(np.float32)


def test_q8_0_equals_the_reference_algorithm():
    w = weights(16, 256, 1)
    w[3, 32:64] = 0.0                       # an all-zero block
    w[5, 7] = 3.0                           # an outlier
    got = kernels.quantize("Q8_0", w)
    want = np.empty_like(got)
    L.oracle().orc_q8_0_quantize(L.fp(w), w.size, L.u8(want))
    assert np.array_equal(got, want)
    with pytest.raises(ValueError):
        kernels.quantize("Q8_0", np.zeros(33, np.float32))      # Q8_0QuantizerTest.kt:66-71


def q4k_fields(b):
    b = b.reshape(-1, 144)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float32).ravel()
    dmin = b[:, 2:4].copy().view(np.float16).astype(np.float32).ravel()
    s = b[:, 4:16].astype(np.int32)
    sc = np.concatenate([s[:, 0:4] & 63, (s[:, 8:12] & 15) | ((s[:, 0:4] >> 6) << 4)], 1)
    mn = np.concatenate([s[:, 4:8] & 63, (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)], 1)
    return d, dmin, sc, mn


def test_q4k_blocks_are_valid_and_round_trip_within_one_step():
    w = weights(8, 1024, 2)
    w[0, :256] = 0.0
    w[1, 256:512] = np.abs(w[1, 256:512])   # all-positive block: min clamps to 0
    q = kernels.quantize("Q4_K", w)
    assert q.size == w.size // 256 * 144
    d, dmin, sc, mn = q4k_fields(q)
    assert np.isfinite(d).all() and np.isfinite(dmin).all() and (d >= 0).all() and (dmin >= 0).all()
    assert sc.max() <= 63 and mn.max() <= 63
    back = L.dequant("Q4_K", q).reshape(-1, 8, 32)
    step = (d[:, None] * sc)[:, :, None]    # one code step of each sub-block
    err = np.abs(back - w.reshape(-1, 8, 32))
    # inside the representable range the error is at most half a step (+ fp16 rounding of d/dmin)
    lo = -(dmin[:, None] * mn)[:, :, None]
    hi = lo + 15 * step
    inside = (w.reshape(-1, 8, 32) >= lo) & (w.reshape(-1, 8, 32) <= hi)
    assert (err[inside] <= np.broadcast_to(0.5 * step + 1e-7, err.shape)[inside] * 1.001).all()
    assert np.sqrt((err ** 2).mean()) / w.std() < 0.09
    assert not back[0].any()
    assert np.array_equal(q, kernels.quantize("Q4_K", w))            # deterministic


def test_q6k_blocks_are_valid_and_round_trip_within_one_step():
    w = weights(8, 1024, 3)
    w[2, 512:768] = 0.0
    q = kernels.quantize("Q6_K", w)
    assert q.size == w.size // 256 * 210
    b = q.reshape(-1, 210)
    d = b[:, 208:210].copy().view(np.float16).astype(np.float32).ravel()
    sc = b[:, 192:208].view(np.int8).astype(np.float32)
    assert np.isfinite(d).all()
    back = L.dequant("Q6_K", q).reshape(-1, 16, 16)
    step = np.abs(d[:, None] * sc)[:, :, None]
    err = np.abs(back - w.reshape(-1, 16, 16))
    inside = np.abs(w.reshape(-1, 16, 16)) <= 31 * step
    assert (err[inside] <= np.broadcast_to(0.5 * step + 1e-7, err.shape)[inside] * 1.001).all()
    assert np.sqrt((err ** 2).mean()) / w.std() < 0.025
    assert np.array_equal(q, kernels.quantize("Q6_K", w))


@pytest.mark.parametrize("enc,tol", [("Q4_K", 0.05), ("Q6_K", 0.012), ("Q8_0", 0.004)])
def test_requantising_a_decoded_tensor_is_nearly_idempotent(enc, tol):
    w = weights(4, 1024, 4)
    once = L.dequant(enc, kernels.quantize(enc, w))
    twice = L.dequant(enc, kernels.quantize(enc, once.reshape(w.shape)))
    assert np.sqrt(((twice - once) ** 2).mean()) / w.std() < tol


def test_to_kernel_order_matches_the_oracle_relayout():
    w = weights(6, 768, 5)
    for enc in ("Q4_K", "Q6_K", "Q8_0"):
        q = kernels.quantize(enc, w)
        _, bs, nb = kernels.ENCODINGS[enc]
        want = np.empty_like(q)
        L.oracle().orc_relayout(L.u8(q), L.u8(want), 6, 768 // bs, nb, 0)
        assert np.array_equal(kernels.to_kernel_order(enc, q, 6, 768 // bs), want)


def test_q4_0_known_answers_of_the_reference_quantizer_test():
    """Q4_0QuantizerTest.kt: 18 bytes per block; round trip within one step (|max| / 8) per block on
    (rng - 0.5) * 4 values; the dominant negative element recovered within 0.05; an all-zero block stays zero."""
    assert kernels.quantize("Q4_0", (0.1 * np.arange(64)).astype(np.float32)).size == 2 * 18
    with pytest.raises(ValueError):
        kernels.quantize("Q4_0", np.zeros(31, np.float32))
    v = ((np.random.default_rng(7).random(32 * 8, dtype=np.float32) - 0.5) * 4).astype(np.float32)
    back = L.dequant("Q4_0", kernels.quantize("Q4_0", v))
    step = np.abs(v.reshape(-1, 32)).max(1, keepdims=True) / 8
    assert (np.abs(back.reshape(-1, 32) - v.reshape(-1, 32)) <= step + 1e-4).all()
    one = np.zeros(32, np.float32); one[5] = -3.7; one[9] = 1.2
    assert abs(L.dequant("Q4_0", kernels.quantize("Q4_0", one))[5] + 3.7) <= 0.05
    assert not L.dequant("Q4_0", kernels.quantize("Q4_0", np.zeros(32, np.float32))).any()
    # the algorithm itself, restated: d = max / -8 (sign of the largest magnitude), code = trunc(x / d + 8.5) in 0..15
    blk = v[:32]
    mx = blk[np.argmax(np.abs(blk))]
    d = np.float32(mx) / np.float32(-8)
    codes = np.clip((blk * (np.float32(1) / d) + np.float32(8.5)).astype(np.int32), 0, 15)
    q = kernels.quantize("Q4_0", blk)
    assert np.array_equal(q[2:] & 0x0F, codes[:16]) and np.array_equal(q[2:] >> 4, codes[16:])
    assert abs(float(q[:2].view(np.float16)[0]) - float(d)) <= abs(float(d)) * 2 ** -10


@pytest.mark.parametrize("enc,levels,rel_rms", [("Q4_0", 16, 0.12), ("Q5_0", 32, 0.06), ("Q5_1", 32, 0.05), ("Q5_K", 32, 0.045)])
def test_q4_0_q5_blocks_round_trip_within_one_step_and_are_deterministic(enc, levels, rel_rms):
    w = weights(8, 1024, 5)
    w[0, :256] = 0.0
    q = kernels.quantize(enc, w)
    assert q.size == w.size // kernels.ENCODINGS[enc][1] * kernels.ENCODINGS[enc][2]
    back = L.dequant(enc, q).reshape(w.shape)
    assert np.isfinite(back).all() and not back[0, :256].any()
    blk = 32
    amax = np.abs(w.reshape(-1, blk)).max(1, keepdims=True)
    rng_ = w.reshape(-1, blk).max(1, keepdims=True) - w.reshape(-1, blk).min(1, keepdims=True)
    step = {"Q4_0": amax / 8, "Q5_0": amax / 16, "Q5_1": rng_ / 31, "Q5_K": rng_ / 31 * 1.2}[enc]
    assert (np.abs(back.reshape(-1, blk) - w.reshape(-1, blk)) <= step * 1.02 + 1e-6).all()
    assert np.sqrt(((back - w) ** 2).mean()) / w.std() < rel_rms
    assert np.array_equal(q, kernels.quantize(enc, w))
    once = L.dequant(enc, kernels.quantize(enc, back))
    assert np.sqrt(((once - back.ravel()) ** 2).mean()) / w.std() < rel_rms
