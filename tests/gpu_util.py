"""Helpers shared by the GPU parity tests (device buffers through torch, checks through the oracle)."""
import numpy as np

from oracle import golden as G

ENCS = ["Q8_0", "Q4_K", "Q6_K"]
MORE_ENCS = ["Q4_0", "Q5_0", "Q5_1", "Q5_K"]          # formats without a quantizer here: tested on seeded valid blocks
SHORT = {"Q8_0": "q8_0", "Q4_K": "q4k", "Q6_K": "q6k", "Q4_0": "q4_0", "Q5_0": "q5_0", "Q5_1": "q5_1", "Q5_K": "q5k"}


def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def random_valid_blocks(enc, nblocks, seed, subnormal_every=0):
    """Random bytes with sane fp16 scale fields (the golden generator's recipe, vectorised); optionally every n-th
    block gets a subnormal fp16 scale to exercise that branch of the fp16 decode."""
    bs, nb, d_off, d2_off = G.PACKED[enc]
    rng = np.random.default_rng(seed)
    b = rng.integers(0, 256, size=(nblocks, nb), dtype=np.uint8)
    d = (rng.random(nblocks, dtype=np.float32) * 0.045 + 0.005).astype(np.float16)
    if subnormal_every:
        d[::subnormal_every] = np.float16(3.0e-6)
    b[:, d_off:d_off + 2] = d.view(np.uint8).reshape(-1, 2)
    if d2_off is not None:
        d2 = (rng.random(nblocks, dtype=np.float32) * 0.02 + 0.005).astype(np.float16)
        b[:, d2_off:d2_off + 2] = d2.view(np.uint8).reshape(-1, 2)
    return b.reshape(-1)


def gaussian_weight(kernels, enc, rows, cols, seed, sigma=0.02):
    w = (np.random.default_rng(seed).standard_normal((rows, cols)) * sigma).astype(np.float32)
    return kernels.quantize(enc, w)


def normalized_err(got, ref, eps=1e-2):
    """max |got - ref| / max(|ref|, eps * ||ref||_inf): relative error with a floor for near-zero entries."""
    ref = np.asarray(ref, np.float64)
    floor = eps * max(np.abs(ref).max(), 1e-30)
    return float((np.abs(np.asarray(got, np.float64) - ref) / np.maximum(np.abs(ref), floor)).max())
