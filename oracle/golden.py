"""Restatement of the reference's golden-test support: seeded inputs and the bit-exact digest.

Follows /root/reference/skainet-backends/skainet-backend-cpu/src/goldenTest/kotlin/sk/ainet/exec/golden/
GoldenSupport.kt: Rng (xorshift64*) :18-31, half() truncating fp32->fp16 :34-42, Packed.block :55-69,
weightBlocks :73-76, rowMajor/blockMajor :79-92, floats :94-97, digest (FNV-1a-64 over raw float
bits, little-endian byte order) :104-112.

Test infrastructure only.
"""
from __future__ import annotations

import struct

import numpy as np

MASK64 = (1 << 64) - 1

# (block_size, bytes_per_block, byte offset of the fp16 `d`, byte offset of a second fp16 or None); the second fp16 is
# `dMin` for the K-quants and `m` for Q5_1 (GoldenSupport.kt:50, :61-66)
PACKED = {
    "Q4_0": (32, 18, 0, None),
    "Q5_0": (32, 22, 0, None),
    "Q5_1": (32, 24, 0, 2),
    "Q8_0": (32, 34, 0, None),
    "Q4_K": (256, 144, 0, 2),
    "Q5_K": (256, 176, 0, 2),
    "Q6_K": (256, 210, 208, None),
}


class Rng:
    """xorshift64* (GoldenSupport.kt:18-31)."""

    def __init__(self, seed: int):
        self.s = 0x9E3779B97F4A7C15 if seed == 0 else seed & MASK64

    def next_long(self) -> int:
        x = self.s
        x ^= x >> 12
        x ^= (x << 25) & MASK64
        x ^= x >> 27
        self.s = x
        return (x * 0x2545F4914F6CDD1D) & MASK64

    def next_byte(self) -> int:
        return self.next_long() >> 56

    def next_float(self) -> np.float32:
        return np.float32(((self.next_long() >> 40) & 0xFFFFFF) / 16777216.0)

    def next_signed(self) -> np.float32:
        return np.float32(self.next_float() * np.float32(2.0) - np.float32(1.0))


def half_trunc(v: np.float32) -> int:
    """GoldenSupport.half: fp32 -> fp16 bits by mantissa truncation (flush below normal range)."""
    bits = struct.unpack("<I", struct.pack("<f", float(v)))[0]
    sign = (bits >> 16) & 0x8000
    expo = ((bits >> 23) & 0xFF) - 127 + 15
    mant = bits & 0x7FFFFF
    if expo <= 0:
        return sign
    if expo >= 31:
        return sign | 0x7C00
    return sign | (expo << 10) | (mant >> 13)


def block(enc: str, rng: Rng) -> bytes:
    """Packed.block: every byte random, then the fp16 fields overwritten with sane scales."""
    _, nbytes, d_off, d2_off = PACKED[enc]
    b = bytearray(rng.next_byte() for _ in range(nbytes))
    d = np.float32(rng.next_float() * np.float32(0.045) + np.float32(0.005))
    d_min = np.float32(rng.next_float() * np.float32(0.02) + np.float32(0.005))
    m = np.float32(rng.next_signed() * np.float32(0.5))  # drawn for every encoding, used only by Q5_1
    b[d_off:d_off + 2] = struct.pack("<H", half_trunc(d))
    if d2_off is not None:
        b[d2_off:d2_off + 2] = struct.pack("<H", half_trunc(m if enc == "Q5_1" else d_min))
    return bytes(b)


def weight_blocks(enc: str, rows: int, blocks_per_row: int, seed: int):
    rng = Rng(seed)
    return [[block(enc, rng) for _ in range(blocks_per_row)] for _ in range(rows)]


def row_major(blocks) -> np.ndarray:
    return np.frombuffer(b"".join(b for row in blocks for b in row), dtype=np.uint8).copy()


def block_major(blocks) -> np.ndarray:
    rows, per_row = len(blocks), len(blocks[0])
    return np.frombuffer(b"".join(blocks[o][bi] for bi in range(per_row) for o in range(rows)),
                         dtype=np.uint8).copy()


def floats(n: int, seed: int, scale: float = 1.0) -> np.ndarray:
    rng = Rng(seed)
    s = np.float32(scale)
    return np.array([rng.next_signed() * s for _ in range(n)], dtype=np.float32)


def fnv1a64(data: bytes) -> int:
    h = 0xCBF29CE484222325
    for byte in data:
        h = ((h ^ byte) * 0x100000001B3) & MASK64
    return h


def digest(values: np.ndarray) -> str:
    """digest(FloatArray): n, FNV-1a-64 over the little-endian raw bits, first four bit patterns."""
    v = np.ascontiguousarray(values, dtype=np.float32).ravel()
    bits = v.view(np.uint32)
    head = ",".join(f"{int(x):08x}" for x in bits[:4])
    return f"n={v.size} fnv={fnv1a64(v.tobytes()):016x} head={head}"


def digest_bytes(data) -> str:
    b = bytes(data)
    return f"n={len(b)} fnv={fnv1a64(b):016x} head={b[:8].hex()}"
