"""Writes tests/golden/ref_vectors.npz: outputs of the reference's own native C kernels (oracle/_ref, compiled by
oracle/Makefile from the sources under /root/reference) on closed-form / seeded inputs.

Run here (the reference is not present on a GPU box):  python tests/golden/make_ref_vectors.py
The vectors pin the oracle's attention, its int8-activation port, its exact kernels for Q4_0 / Q5_0 / Q5_1 / Q5_K and its
bf16 / fp16 dense matmul where the reference library is absent.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from oracle import golden as G  # noqa: E402
from oracle import lib as L  # noqa: E402
from test_oracle_golden import SDPA_GRID, narrow_inputs, sdpa_inputs  # noqa: E402


def main():
    ref = L.ref()
    assert ref is not None, "build oracle/_ref first: make -C oracle ref"
    out = {}
    for i, (h, hkv, sq, skv, causal, use_len, win, rc) in enumerate(SDPA_GRID):
        q, k, v = sdpa_inputs(3, h, hkv, sq, skv, 8)
        lengths = np.array([skv, (skv + 1) // 2, 1], np.int32) if use_len else None
        out[f"sdpa/{i}"] = L.sdpa(q, k, v, 1.0 / np.sqrt(8), causal, win, rc, lengths, lib=ref)
    for enc, short in (("Q8_0", "q8_0"), ("Q4_K", "q4k"), ("Q6_K", "q6k")):
        bs = G.PACKED[enc][0]
        n, nblocks = 6, 3
        w = G.row_major(G.weight_blocks(enc, n, nblocks, 0x5EED0010))
        x = G.floats(nblocks * bs, 0x5EED0011)
        y = np.empty(n, np.float32)
        getattr(ref, f"skainet_{short}_matmul_rm")(L.fp(x), 0, L.u8(w), 0, nblocks * bs, n, L.fp(y), 0)
        out[f"native_rm/{enc}"] = y
    # exact fp32 kernels of the reference library (no int8 activations on these formats)
    for enc in ("Q4_0", "Q5_0", "Q5_1", "Q5_K"):
        bs = G.PACKED[enc][0]
        n, nblocks = 6, 3
        w = G.row_major(G.weight_blocks(enc, n, nblocks, 0x5EED0010))
        x = G.floats(nblocks * bs, 0x5EED0011)
        y = np.empty(n, np.float32)
        getattr(ref, f"skainet_{L._SHORT[enc]}_matmul_rm")(L.fp(x), 0, L.u8(w), 0, nblocks * bs, n, L.fp(y), 0)
        out[f"native_rm/{enc}"] = y
    for kind in ("bf16", "fp16"):
        a, b, m, n, k = narrow_inputs(kind)
        out[f"narrow/{kind}"] = L.narrow_matmul(kind, a, b, m, n, k, lib=ref)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
