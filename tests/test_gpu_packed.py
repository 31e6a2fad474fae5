"""GPU parity, packed weights: bit-exact decode and the dequant-GEMV kernels against the exact-fp32 oracle.

Tolerances (stated by the task): decode bit-exact; GEMV (fp32 path) max relative error <= 1e-3, measured as
|got - ref| / max(|ref|, 1e-2 * ||ref||_inf) -- per-row relative error of a near-zero row is unbounded, the
reference's own parity test says the same (NativeQ4KMatmulKernelParityTest.kt:75-83).
"""
import json
import os

import numpy as np
import pytest

from oracle import golden as G
from oracle import lib as L
from gpu_util import ENCS, MORE_ENCS, dev, gaussian_weight, normalized_err, random_valid_blocks

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
GOLDENS = json.load(open(os.path.join(HERE, "golden", "reference_goldens.json")))
GEMV_TOL = 1e-3


def gpu_dequant(kernels, torch, enc, packed, rows, cols):
    w = kernels.DeviceWeight.upload(enc, packed, rows, cols)
    out = torch.empty(rows * cols, dtype=torch.float32, device="cuda")
    w.dequantize(out)
    return out.cpu().numpy()


@pytest.mark.parametrize("enc", ENCS)
def test_decode_reproduces_the_reference_golden_digest(hip_backend, torch_cuda, enc):
    bs = G.PACKED[enc][0]
    packed = G.row_major(G.weight_blocks(enc, 4, 3, 0x5EED0001))
    got = gpu_dequant(hip_backend, torch_cuda, enc, packed, 4, 3 * bs)
    assert G.digest(got) == GOLDENS[f"decode/{enc}"]


@pytest.mark.parametrize("enc", ENCS)
def test_decode_bit_exact_on_random_and_quantised_blocks(hip_backend, torch_cuda, enc):
    bs = G.PACKED[enc][0]
    rows, cols = 37, 5 * 256
    for packed in (random_valid_blocks(enc, rows * cols // bs, 11, subnormal_every=7),
                   gaussian_weight(hip_backend, enc, rows, cols, 12)):
        got = gpu_dequant(hip_backend, torch_cuda, enc, packed, rows, cols)
        assert np.array_equal(got.view(np.uint32), L.dequant(enc, packed).view(np.uint32))


@pytest.mark.parametrize("enc,rows,cols", [("Q4_K", 11008, 4096), ("Q8_0", 4096, 4096), ("Q6_K", 8000, 4096)])
def test_decode_bit_exact_at_config_sizes(hip_backend, torch_cuda, enc, rows, cols):
    packed = gaussian_weight(hip_backend, enc, rows, cols, 21)
    got = gpu_dequant(hip_backend, torch_cuda, enc, packed, rows, cols)
    want = L.dequant(enc, packed)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("enc", ENCS)
def test_embedding_row_gather_is_the_decode_of_those_rows(hip_backend, torch_cuda, enc):
    rows, cols = 50, 512
    packed = gaussian_weight(hip_backend, enc, rows, cols, 5)
    ids = np.array([3, 49, 0, 3, 17], np.int32)
    w = hip_backend.DeviceWeight.upload(enc, packed, rows, cols)
    out = torch_cuda.empty(len(ids) * cols, dtype=torch_cuda.float32, device="cuda")
    w.dequantize_rows(dev(torch_cuda, ids), len(ids), out)
    want = L.dequant(enc, packed).reshape(rows, cols)[ids]
    assert np.array_equal(out.cpu().numpy().reshape(len(ids), cols).view(np.uint32), want.view(np.uint32))


def gpu_matmul(kernels, torch, enc, packed, n, k, x, kind=0, order=0):
    w = kernels.DeviceWeight.upload(enc, packed, n, k, order)
    m = x.shape[0]
    y = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
    w.matmul(dev(torch, x), m, y, kind)
    return y.cpu().numpy()


@pytest.mark.parametrize("enc", ENCS)
def test_gemv_on_the_reference_golden_inputs(hip_backend, torch_cuda, enc):
    """ScalarKernelGoldenTest inputs: the oracle reproduces the golden digest bit for bit (test_oracle_golden), the HIP
    kernel sums in another order and must agree within the fp32-path tolerance -- from both block orders."""
    bs = G.PACKED[enc][0]
    blocks = G.weight_blocks(enc, 4, 3, 0x5EED0002)
    x = G.floats(3 * 3 * bs, 0x5EED0002 + 100).reshape(3, 3 * bs)
    want = L.gemv(enc, x, G.row_major(blocks), 4)
    assert G.digest(want) == GOLDENS[f"scalar-matmul/{enc}"]
    got_rm = gpu_matmul(hip_backend, torch_cuda, enc, G.row_major(blocks), 4, 3 * bs, x)
    got_bm = gpu_matmul(hip_backend, torch_cuda, enc, G.block_major(blocks), 4, 3 * bs, x, order=1)
    assert normalized_err(got_rm, want) <= GEMV_TOL
    assert np.array_equal(got_rm, got_bm)   # the upload permutation changes nothing


@pytest.mark.parametrize("enc", ENCS)
@pytest.mark.parametrize("n,k,m", [(1, 256, 1), (3, 512, 2), (63, 768, 3), (65, 2048, 4), (130, 2304, 5), (1000, 4096, 8),
                                   (257, 11008, 1), (96, 14336, 2), (40, 16640, 1)])
def test_gemv_ragged_shapes_and_batches(hip_backend, torch_cuda, enc, n, k, m):
    bs = G.PACKED[enc][0]
    packed = random_valid_blocks(enc, n * k // bs, 100 + n)
    x = np.random.default_rng(n + k).standard_normal((m, k)).astype(np.float32)
    got = gpu_matmul(hip_backend, torch_cuda, enc, packed, n, k, x)
    want = L.gemv(enc, x, packed, n)
    assert not np.isnan(got).any()
    assert normalized_err(got, want) <= GEMV_TOL


@pytest.mark.parametrize("enc,n,k,batches", [("Q8_0", 4096, 4096, (1,)), ("Q4_K", 11008, 4096, (1, 4, 8)),
                                             ("Q6_K", 32000, 4096, (1,)), ("Q4_K", 4096, 14336, (1,))])
def test_gemv_at_config_sizes(hip_backend, torch_cuda, enc, n, k, batches):
    packed = gaussian_weight(hip_backend, enc, n, k, 31)
    for m in batches:
        x = np.random.default_rng(40 + m).standard_normal((m, k)).astype(np.float32)
        got = gpu_matmul(hip_backend, torch_cuda, enc, packed, n, k, x)
        want = L.gemv(enc, x, packed, n)
        err = normalized_err(got, want)
        print(f"{enc} {n}x{k} batch {m}: normalized max err {err:.2e}")
        assert err <= GEMV_TOL


@pytest.mark.parametrize("mode", ["slot-fp32", "rows-fp32", "mfma-i8"])
@pytest.mark.parametrize("n,k,m", [(11008, 4096, 1), (11008, 4096, 2), (4096, 14336, 1), (2050, 8448, 1), (1537, 16640, 1), (6144, 8192, 1),
                                   (1000, 11008, 1), (77, 2304, 2), (5, 256, 1), (1030, 1024, 1), (7, 2048, 1), (515, 3072, 1),
                                   (2052, 5120, 1), (300, 16384, 1), (28672, 4096, 1), (36000, 1024, 1), (4096, 12288, 1)])
def test_q4k_decode_kernel_variants_agree_with_the_oracle(hip_backend, torch_cuda, mode, n, k, m):
    """The Q4_K decode kernels (the generic slot kernel, the fp32 row-streaming kernel and the integer matrix-core
    kernel that takes one-row products with K in whole slices of 1024) are held to the same bound against the
    exact-fp32 oracle, on quantised Gaussian weights and on random valid blocks with large scales. The long-row shapes
    (4096 x 14336; 2050 x 8448: 33 super-blocks per row, a ragged last workgroup; 1537 x 16640: 65 super-blocks, two
    passes per wave, four rows per workgroup; 6144 x 8192: twelve) take the form of the row kernel that splits K over the
    waves of a workgroup; K of 1 to 16 slices, row counts that are not a multiple of 4, more quads than one round of
    workgroups holds (28672 and 36000 rows) exercise the matrix-core kernel's slice and quad bookkeeping."""
    hip_backend.set_tuning("q4k_rows_enable", 0 if mode == "slot-fp32" else 1)
    hip_backend.set_tuning("q4k_mfma_enable", 1 if mode == "mfma-i8" else 0)
    try:
        for packed in (gaussian_weight(hip_backend, "Q4_K", n, k, 71), random_valid_blocks("Q4_K", n * k // 256, 72)):
            x = np.random.default_rng(73 + m).standard_normal((m, k)).astype(np.float32)
            x[0, :64] = 0.0          # a constant slice (zero range) and an outlier
            x[0, 100] = 37.5
            got = gpu_matmul(hip_backend, torch_cuda, "Q4_K", packed, n, k, x)
            err = normalized_err(got, L.gemv("Q4_K", x, packed, n))
            print(f"{mode} {n}x{k} m={m}: {err:.2e}")
            assert err <= GEMV_TOL
    finally:
        hip_backend.set_tuning("q4k_rows_enable", 1)
        hip_backend.set_tuning("q4k_mfma_enable", 1)


@pytest.mark.parametrize("n", [8, 37, 515, 4096, 11008, 28672, 40000])
def test_q4k_one_row_kernel_with_two_teams_of_waves(hip_backend, torch_cuda, n):
    """K = 4096: two teams of four waves per workgroup (the teams split the row quads and each prepares half of a slice's
    activation planes) against one team. Every (slice, quad) partial sum is formed by the same instructions in the same
    order either way, so the results are the same bits: plain, with a residual, with the RMSNorm prologue, with SwiGLU."""
    k = 4096
    packed = gaussian_weight(hip_backend, "Q4_K", n, k, 61) if n <= 11008 else random_valid_blocks("Q4_K", n * k // 256, 62)
    rng = np.random.default_rng(63 + n)
    x = rng.standard_normal((1, k)).astype(np.float32)
    gain = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    res = rng.standard_normal((1, n)).astype(np.float32)
    w = hip_backend.DeviceWeight.upload("Q4_K", packed, n, k)
    xd, gd, rd = dev(torch_cuda, x), dev(torch_cuda, gain), dev(torch_cuda, res)

    def run(teams):
        hip_backend.set_tuning("q4k_mfma_teams", teams)
        outs = []
        for kw in ({}, {"residual": rd, "epilogue": 1}, {"gain": gd, "eps": 1e-5}, {"gain": gd, "eps": 1e-5, "epilogue": 2}):
            cols = n // 2 if kw.get("epilogue") == 2 else n
            if kw.get("epilogue") == 2 and n % 2:
                continue
            y = torch_cuda.full((1, cols), float("nan"), dtype=torch_cuda.float32, device="cuda")
            w.matmul_fused(xd, 1, y, **kw)
            assert hip_backend.last_kernel() == "q4k_gemv_mfma_kernel"
            outs.append(y.cpu().numpy())
        return outs

    try:
        one, two = run(1), run(2)
    finally:
        hip_backend.set_tuning("q4k_mfma_teams", 0)
    assert normalized_err(one[0], L.gemv("Q4_K", x, packed, n)) <= GEMV_TOL
    for a, b in zip(one, two):
        assert not np.isnan(b).any()
        assert np.array_equal(a, b)


@pytest.mark.parametrize("n,k", [(4096, 14336), (2050, 8192), (517, 16384), (64, 12288)])
def test_q4k_one_row_kernel_with_eight_waves_on_long_rows(hip_backend, torch_cuda, n, k):
    """Rows of 8192 elements and more without a prologue: K split over eight waves instead of four (another order of the
    fp32 sums), plain and with a residual, against the oracle and against the four-wave form."""
    packed = gaussian_weight(hip_backend, "Q4_K", n, k, 51)
    rng = np.random.default_rng(52 + n)
    x = rng.standard_normal((1, k)).astype(np.float32)
    res = rng.standard_normal((1, n)).astype(np.float32)
    w = hip_backend.DeviceWeight.upload("Q4_K", packed, n, k)
    xd, rd = dev(torch_cuda, x), dev(torch_cuda, res)
    want = L.gemv("Q4_K", x, packed, n)
    outs = {}
    try:
        for eight in (1, 0):
            hip_backend.set_tuning("q4k_mfma_waves8", eight)
            y = torch_cuda.full((1, n), float("nan"), dtype=torch_cuda.float32, device="cuda")
            w.matmul_fused(xd, 1, y)
            assert hip_backend.last_kernel() == "q4k_gemv_mfma_kernel"
            yr = torch_cuda.full((1, n), float("nan"), dtype=torch_cuda.float32, device="cuda")
            w.matmul_fused(xd, 1, yr, residual=rd, epilogue=1)
            outs[eight] = (y.cpu().numpy(), yr.cpu().numpy())
            assert normalized_err(outs[eight][0], want) <= GEMV_TOL
            assert normalized_err(outs[eight][1], want + res) <= GEMV_TOL
    finally:
        hip_backend.set_tuning("q4k_mfma_waves8", 1)
    assert normalized_err(outs[1][0], outs[0][0]) <= 2e-5


@pytest.mark.parametrize("slot64", [1, 0])
@pytest.mark.parametrize("n,k", [(8000, 4096), (515, 4096), (70, 768), (33, 256), (257, 14336), (3, 16640)])
def test_q6k_batch1_slot_variants_agree_with_the_oracle(hip_backend, torch_cuda, slot64, n, k):
    """Q6_K at batch 1 with the 64-weight slot (16-byte code loads, the default) and with the 32-weight slot of the
    batched kernel: the same bound against the exact-fp32 oracle, on quantised Gaussian weights and on random valid
    blocks; rows of one super-block, rows longer than one wave pass, ragged last workgroups."""
    hip_backend.set_tuning("q6k_slot64", slot64)
    hip_backend.set_tuning("gemv_stream_enable", 0)      # the row kernel's two slot shapes are what this test compares
    try:
        for packed in (gaussian_weight(hip_backend, "Q6_K", n, k, 81), random_valid_blocks("Q6_K", n * k // 256, 82)):
            x = np.random.default_rng(83).standard_normal((1, k)).astype(np.float32)
            x[0, :64] = 0.0
            x[0, 100] = 37.5
            got = gpu_matmul(hip_backend, torch_cuda, "Q6_K", packed, n, k, x)
            err = normalized_err(got, L.gemv("Q6_K", x, packed, n))
            print(f"slot64={slot64} {n}x{k}: {err:.2e}")
            assert err <= GEMV_TOL
    finally:
        hip_backend.set_tuning("q6k_slot64", 1)
        hip_backend.set_tuning("gemv_stream_enable", 1)


STREAM_ENCS = ["Q8_0", "Q4_0", "Q5_0", "Q5_1"]


@pytest.mark.parametrize("enc", STREAM_ENCS)
@pytest.mark.parametrize("n,k", [(4096, 4096), (11008, 4096), (1000, 4096), (1027, 2048), (70, 768), (33, 256), (5000, 1024), (3, 4096),
                                 (2100, 8192)])
def test_one_row_products_streamed_through_lds(hip_backend, torch_cuda, enc, n, k):
    """One activation row against the formats of 32-element blocks: rows whose byte length is a multiple of 16 and
    that have at most 128 blocks take the kernel that streams each wave's rows through LDS; the others stay on the row
    kernel. Both against the exact-fp32 oracle (1e-3), and against each other (same products, another
    summation order). Shapes: one, two and many units per wave, ragged last waves and workgroups, fewer rows than waves,
    rows shorter than a wave's 64 slots."""
    bs, bb = G.PACKED[enc][0], G.PACKED[enc][1]
    row_bytes = k // bs * bb
    eligible = row_bytes % 16 == 0 and k // 32 <= 128
    packed = gaussian_weight(hip_backend, enc, n, k, 61) if n * k >= 1 << 22 else random_valid_blocks(enc, n * k // bs, 62 + n)
    x = np.random.default_rng(63 + k).standard_normal((1, k)).astype(np.float32)
    x[0, 5] = -41.0
    want = L.gemv(enc, x, packed, n)
    try:
        hip_backend.set_tuning("q8_0_mfma_enable", 0)       # (Q8_0 rows of 1024 to 4096 elements would take the matrix-core kernel)
        got = gpu_matmul(hip_backend, torch_cuda, enc, packed, n, k, x)
        assert hip_backend.last_kernel() == ("gemv_stream_kernel" if eligible else "gemv_kernel")
        assert not np.isnan(got).any()
        assert normalized_err(got, want) <= GEMV_TOL
        hip_backend.set_tuning("gemv_stream_enable", 0)
        rows = gpu_matmul(hip_backend, torch_cuda, enc, packed, n, k, x)
        assert hip_backend.last_kernel() == "gemv_kernel"
    finally:
        hip_backend.set_tuning("gemv_stream_enable", 1)
        hip_backend.set_tuning("q8_0_mfma_enable", 1)
    assert normalized_err(got, rows) <= 2e-5


@pytest.mark.parametrize("n,k", [(4096, 4096), (11008, 4096), (1000, 4096), (1027, 2048), (5000, 1024), (3, 4096), (1, 1024), (17, 3072),
                                 (40000, 1024)])
def test_q8_0_one_row_on_the_integer_matrix_cores(hip_backend, torch_cuda, n, k):
    """One activation row against Q8_0, K a multiple of 1024 up to 4096: the int8 codes go onto v_mfma_i32_4x4x4_16b_i8 as
    they lie, the activations as 22-bit fixed point per 64-element group. Against the exact-fp32 oracle (1e-3) and the
    fp32 streaming kernel; shapes with one to four K slices, fewer quads than the four requested up front, ragged
    quads, ring refills (more than four quads per workgroup) and more than one round of workgroups. Codes at the
    extremes against a constant activation vector: the digit sums are at their largest."""
    packed = gaussian_weight(hip_backend, "Q8_0", n, k, 61) if n * k >= 1 << 22 else random_valid_blocks("Q8_0", n * k // 32, 62 + n)
    x = np.random.default_rng(63 + k).standard_normal((1, k)).astype(np.float32)
    x[0, 5] = -41.0
    want = L.gemv("Q8_0", x, packed, n)
    got = gpu_matmul(hip_backend, torch_cuda, "Q8_0", packed, n, k, x)
    assert hip_backend.last_kernel() == "q8_0_gemv_mfma_kernel"
    assert not np.isnan(got).any()
    err = normalized_err(got, want)
    print(f"Q8_0 {n}x{k} on the matrix cores: {err:.2e}")
    assert err <= GEMV_TOL
    try:
        hip_backend.set_tuning("q8_0_mfma_enable", 0)
        fp32 = gpu_matmul(hip_backend, torch_cuda, "Q8_0", packed, n, k, x)
        assert hip_backend.last_kernel() == "gemv_stream_kernel"
    finally:
        hip_backend.set_tuning("q8_0_mfma_enable", 1)
    assert normalized_err(got, fp32) <= 1e-4
    if n <= 1027:
        # saturated codes (+127 / -127 rows) against constant activations: every digit sum at its extreme
        blocks = np.frombuffer(packed, np.uint8).reshape(n, k // 32, 34).copy()
        blocks[0::2, :, 2:] = 127
        blocks[1::2, :, 2:] = 129                                   # -127
        sat = blocks.reshape(-1)
        for xc in (np.full((1, k), 3.25, np.float32), np.full((1, k), -1e-3, np.float32)):
            got = gpu_matmul(hip_backend, torch_cuda, "Q8_0", sat, n, k, xc)
            assert normalized_err(got, L.gemv("Q8_0", xc, sat, n)) <= GEMV_TOL


def test_q8_0_matrix_core_kernel_keeps_non_finite_activations_loud(hip_backend, torch_cuda):
    """The exact-fp32 product propagates a NaN or an infinity among the activations into every output; the fixed-point
    kernel must not turn it into a finite number: the group's scale becomes NaN. A group of subnormal activations
    contributes (next to) nothing, as in fp32."""
    n, k = 64, 2048
    packed = random_valid_blocks("Q8_0", n * k // 32, 7)
    rng = np.random.default_rng(8)
    for bad in (np.nan, np.inf, -np.inf):
        x = rng.standard_normal((1, k)).astype(np.float32)
        x[0, 700] = bad
        got = gpu_matmul(hip_backend, torch_cuda, "Q8_0", packed, n, k, x)
        assert hip_backend.last_kernel() == "q8_0_gemv_mfma_kernel"
        assert not np.isfinite(got).any(), bad
    x = rng.standard_normal((1, k)).astype(np.float32)
    x[0, 128:192] = np.float32(1e-41) * rng.standard_normal(64).astype(np.float32)      # one group of subnormals
    got = gpu_matmul(hip_backend, torch_cuda, "Q8_0", packed, n, k, x)
    assert np.isfinite(got).all() and normalized_err(got, L.gemv("Q8_0", x, packed, n)) <= GEMV_TOL


@pytest.mark.parametrize("n,k,m", [(5, 256, 3), (25, 1280, 8), (77, 2304, 7), (1000, 11008, 4), (11008, 4096, 6), (4096, 14336, 8),
                                   (130, 4096, 9), (64, 1024, 11)])
def test_q4k_three_to_eight_rows_on_the_matrix_instruction(hip_backend, torch_cuda, n, k, m):
    """3 to 8 activation rows take the 4x4x4 bf16 MFMA kernel (9 and 11 rows: 8 + the rest). Codes are exact in bf16 and
    an activation enters as bf16 hi + bf16 lo (16 to 17 significant bits, exact products, fp32 sums): the one-row bound
    holds with room, and every batch row equals that row run alone (exact fp32) to the split's precision -- 2^-17 per
    term, seen through this metric's floor of 1 % of the largest output."""
    for packed in (gaussian_weight(hip_backend, "Q4_K", n, k, 81), random_valid_blocks("Q4_K", n * k // 256, 82)):
        x = np.random.default_rng(83 + m).standard_normal((m, k)).astype(np.float32)
        x[1, :64] = 0.0
        x[m - 1, 100] = -41.0
        got = gpu_matmul(hip_backend, torch_cuda, "Q4_K", packed, n, k, x)
        assert got.shape == (m, n) and not np.isnan(got).any()
        assert normalized_err(got, L.gemv("Q4_K", x, packed, n)) <= GEMV_TOL
        hip_backend.set_tuning("q4k_mfma_enable", 0)          # "alone" on the exact-fp32 row kernel
        try:
            alone = gpu_matmul(hip_backend, torch_cuda, "Q4_K", packed, n, k, x[m - 1:m])
        finally:
            hip_backend.set_tuning("q4k_mfma_enable", 1)
        assert normalized_err(got[m - 1], alone[0]) <= 3e-4


@pytest.mark.parametrize("n,m", [(4, 3), (5, 4), (37, 5), (130, 8), (1027, 7), (11008, 4), (11008, 8), (28672, 3), (40000, 8)])
def test_q4k_three_to_eight_rows_streamed_through_lds_at_k_4096(hip_backend, torch_cuda, n, m):
    """K = 4096: the batched kernel whose weight arrives through an LDS ring (one K slice per wave), on row counts that
    leave ragged quads, ragged groups of quads and more than one round of workgroups; against the oracle and against the
    register-fed kernel of the same arithmetic (another order of the fp32 sums)."""
    k = 4096
    packed = gaussian_weight(hip_backend, "Q4_K", n, k, 91) if n <= 11008 else random_valid_blocks("Q4_K", n * k // 256, 92)
    x = np.random.default_rng(93 + m + n).standard_normal((m, k)).astype(np.float32)
    x[m - 1, 7] = 33.0
    try:
        hip_backend.set_tuning("q4k_wide_enable", 0)
        got = gpu_matmul(hip_backend, torch_cuda, "Q4_K", packed, n, k, x)
        assert hip_backend.last_kernel() == "q4k_gemv_quads_stream_kernel"
        assert got.shape == (m, n) and not np.isnan(got).any()
        rows = np.unique(np.concatenate([np.arange(min(n, 40)), np.arange(max(0, n - 40), n)]))
        want = L.gemv("Q4_K", x, packed.reshape(n, -1)[rows].reshape(-1), len(rows))
        assert normalized_err(got[:, rows], want) <= GEMV_TOL
        hip_backend.set_tuning("q4k_quads_stream_enable", 0)
        fed = gpu_matmul(hip_backend, torch_cuda, "Q4_K", packed, n, k, x)
        assert hip_backend.last_kernel() == "q4k_gemv_quads_kernel"
    finally:
        hip_backend.set_tuning("q4k_quads_stream_enable", 1)
        hip_backend.set_tuning("q4k_wide_enable", 1)
    assert normalized_err(got, fed) <= 2e-5


@pytest.mark.parametrize("n,m", [(1, 3), (4, 3), (5, 4), (16, 8), (17, 5), (37, 5), (130, 8), (1027, 7), (4096, 6), (11008, 3), (11008, 4),
                                 (11008, 8), (28672, 5), (40000, 8)])
def test_q4k_three_to_eight_rows_on_the_16x16x32_matrix_instruction(hip_backend, torch_cuda, n, m):
    """K = 4096: the batched kernel on v_mfma_f32_16x16x32_bf16 (16 weight rows x one sub-block x 8 batch rows' hi and lo
    parts per instruction, eight K slices per workgroup), on row counts that leave ragged units of 16 rows, workgroups
    with one to eight units (fewer than the three requested up front, and more: the ring is refilled) and more than one
    round of workgroups; against the oracle on the first and last rows, and against the 4x4x4 kernel of the same
    arithmetic over the whole product (another order of the fp32 sums)."""
    k = 4096
    packed = gaussian_weight(hip_backend, "Q4_K", n, k, 91) if n <= 11008 else random_valid_blocks("Q4_K", n * k // 256, 92)
    x = np.random.default_rng(93 + m + n).standard_normal((m, k)).astype(np.float32)
    x[m - 1, 7] = 33.0
    x[1, 512:576] = 0.0
    try:
        hip_backend.set_tuning("q4k_wide_min_batch", 3)      # by itself the launcher takes this kernel from 5 rows on
        got = gpu_matmul(hip_backend, torch_cuda, "Q4_K", packed, n, k, x)
        assert hip_backend.last_kernel() == "q4k_gemv_wide_kernel"
        assert got.shape == (m, n) and not np.isnan(got).any()
        rows = np.unique(np.concatenate([np.arange(min(n, 40)), np.arange(max(0, n - 40), n)]))
        want = L.gemv("Q4_K", x, packed.reshape(n, -1)[rows].reshape(-1), len(rows))
        assert normalized_err(got[:, rows], want) <= GEMV_TOL
        hip_backend.set_tuning("q4k_wide_enable", 0)
        quads = gpu_matmul(hip_backend, torch_cuda, "Q4_K", packed, n, k, x)
        assert hip_backend.last_kernel() in ("q4k_gemv_quads_stream_kernel", "q4k_gemv_quads_kernel")
    finally:
        hip_backend.set_tuning("q4k_wide_enable", 1)
        hip_backend.set_tuning("q4k_wide_min_batch", 5)
    assert normalized_err(got, quads) <= 3e-4      # two orders of fp32 sums, seen through this metric's floor of 1 % of the largest output


def test_gemv_is_linear_and_deterministic_at_full_size(hip_backend, torch_cuda):
    """Size-independent properties at the benchmark shape: y(a*x1 + x2) == a*y(x1) + y(x2) within rounding; two runs agree bit for bit."""
    n, k = 11008, 4096
    packed = gaussian_weight(hip_backend, "Q4_K", n, k, 33)
    rng = np.random.default_rng(7)
    x1, x2 = rng.standard_normal((1, k)).astype(np.float32), rng.standard_normal((1, k)).astype(np.float32)
    y1 = gpu_matmul(hip_backend, torch_cuda, "Q4_K", packed, n, k, x1)
    y2 = gpu_matmul(hip_backend, torch_cuda, "Q4_K", packed, n, k, x2)
    y12 = gpu_matmul(hip_backend, torch_cuda, "Q4_K", packed, n, k, 2.0 * x1 + x2)
    assert normalized_err(y12, 2.0 * y1.astype(np.float64) + y2) <= 1e-4
    assert np.array_equal(y1, gpu_matmul(hip_backend, torch_cuda, "Q4_K", packed, n, k, x1))
    # a batch row equals the same row run alone
    yb = gpu_matmul(hip_backend, torch_cuda, "Q4_K", packed, n, k, np.concatenate([x1, x2, x1, x2]))
    assert normalized_err(yb[1], y2[0]) <= 5e-4   # another kernel: activations as bf16 hi + lo, another summation order


@pytest.mark.parametrize("enc", ENCS)
def test_spi_kernels_on_host_arrays(hip_backend, torch_cuda, enc):
    """The KernelProvider accessors: input-block-major weight, offsets honoured, argument errors raised first."""
    provider = hip_backend.HipKernelProvider()
    assert provider.is_available() and provider.supports("matmul", ["Float32", enc])
    kernel = {"Q4_K": provider.matmul_q4k, "Q6_K": provider.matmul_q6k, "Q8_0": provider.matmul_q8_0}[enc]()
    bs, nb = G.PACKED[enc][0], G.PACKED[enc][1]
    n, nblocks = 70, 4
    k = nblocks * bs
    blocks = G.weight_blocks(enc, n, nblocks, 0x5EED0020)
    x = G.floats(k, 0x5EED0021)
    want = L.gemv(enc, x, G.row_major(blocks), n)
    pad_x, pad_w, pad_y = 5, 2 * nb, 3
    xin = np.concatenate([np.full(pad_x, 9, np.float32), x])
    wbm = np.concatenate([np.full(pad_w, 0xAB, np.uint8), G.block_major(blocks)])
    out = np.full(pad_y + n + 2, 7, np.float32)
    kernel.matmul(xin, pad_x, wbm, pad_w, k, n, out, pad_y)
    assert (out[:pad_y] == 7).all() and (out[pad_y + n:] == 7).all()
    assert normalized_err(out[pad_y:pad_y + n], want) <= GEMV_TOL
    out2 = np.zeros(n, np.float32)
    kernel.matmul_row_major(x, 0, G.row_major(blocks), 0, k, n, out2, 0)
    assert np.array_equal(out2, out[pad_y:pad_y + n])
    with pytest.raises(ValueError):
        kernel.matmul(x, 0, wbm, 0, k - 1, n, out, 0)
    # the view kernel: all rows at once against a GGUF-ordered weight, weight cached on the device
    vk = hip_backend.HipRowMajorMatmulKernel(enc)
    a = G.floats(3 * k, 0x5EED0022).reshape(3, k)
    o = np.zeros((3, n), np.float32)
    wrm = G.row_major(blocks)
    vk.run(a, wrm, n, o)
    vk.run(a, wrm, n, o)
    assert len(vk._cache) == 1
    assert normalized_err(o, L.gemv(enc, a, wrm, n)) <= GEMV_TOL


# ---- the remaining packed formats of the provider SPI (Q4_0, Q5_0, Q5_1, Q5_K): same bars, seeded valid blocks ----
@pytest.mark.parametrize("enc", MORE_ENCS)
def test_more_formats_decode_reproduces_the_reference_golden_digest_and_is_bit_exact(hip_backend, torch_cuda, enc):
    bs = G.PACKED[enc][0]
    blocks = G.weight_blocks(enc, 4, 3, 0x5EED0001)
    got = gpu_dequant(hip_backend, torch_cuda, enc, G.row_major(blocks), 4, 3 * bs)
    assert G.digest(got) == GOLDENS[f"decode/{enc}"]
    for rows, cols, seed in ((7, 2 * bs, 1), (129, 5 * bs, 2), (1024, 4096, 3)):
        packed = random_valid_blocks(enc, rows * cols // bs, 500 + seed, subnormal_every=7)
        got = gpu_dequant(hip_backend, torch_cuda, enc, packed, rows, cols)
        assert np.array_equal(got.view(np.uint32), L.dequant(enc, packed).view(np.uint32))
    # packed embedding lookup: a gather of rows decodes to those rows
    rows, cols = 50, 3 * bs
    packed = random_valid_blocks(enc, rows * cols // bs, 510)
    w = hip_backend.DeviceWeight.upload(enc, packed, rows, cols)
    ids = np.array([49, 0, 7, 7, 31], np.int32)
    out = torch_cuda.empty((len(ids), cols), dtype=torch_cuda.float32, device="cuda")
    w.dequantize_rows(dev(torch_cuda, ids), len(ids), out)
    want = L.dequant(enc, packed).reshape(rows, cols)[ids]
    assert np.array_equal(out.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("enc", MORE_ENCS)
def test_more_formats_gemv_on_the_reference_golden_inputs(hip_backend, torch_cuda, enc):
    bs = G.PACKED[enc][0]
    blocks = G.weight_blocks(enc, 4, 3, 0x5EED0002)
    x = G.floats(3 * 3 * bs, 0x5EED0002 + 100).reshape(3, 3 * bs)
    want = L.gemv(enc, x, G.row_major(blocks), 4)
    assert G.digest(want) == GOLDENS[f"scalar-matmul/{enc}"]
    got_rm = gpu_matmul(hip_backend, torch_cuda, enc, G.row_major(blocks), 4, 3 * bs, x)
    got_bm = gpu_matmul(hip_backend, torch_cuda, enc, G.block_major(blocks), 4, 3 * bs, x, order=1)
    assert normalized_err(got_rm, want) <= GEMV_TOL
    assert np.array_equal(got_rm, got_bm)


@pytest.mark.parametrize("enc", MORE_ENCS)
@pytest.mark.parametrize("n,k,m", [(1, 256, 1), (3, 512, 2), (65, 2048, 4), (130, 2304, 5), (1000, 4096, 1), (257, 11008, 1),
                                   (40, 16640, 3), (300, 1024, 24)])
def test_more_formats_gemv_ragged_shapes_and_batches(hip_backend, torch_cuda, enc, n, k, m):
    """Exact-fp32 products through the row kernels at every row count (kind 0 forces them; 24 rows = six passes)."""
    bs = G.PACKED[enc][0]
    packed = random_valid_blocks(enc, n * k // bs, 600 + n)
    x = np.random.default_rng(n + k).standard_normal((m, k)).astype(np.float32)
    x[0, :64] = 0.0
    got = gpu_matmul(hip_backend, torch_cuda, enc, packed, n, k, x, kind=0)
    assert not np.isnan(got).any()
    assert normalized_err(got, L.gemv(enc, x, packed, n)) <= GEMV_TOL


@pytest.mark.parametrize("enc", MORE_ENCS)
def test_more_formats_spi_kernels_on_host_arrays(hip_backend, torch_cuda, enc):
    provider = hip_backend.HipKernelProvider()
    assert provider.supports("matmul", ["Float32", enc])
    kernel = {"Q4_0": provider.matmul_q4_0, "Q5_0": provider.matmul_q5_0, "Q5_1": provider.matmul_q5_1,
              "Q5_K": provider.matmul_q5k}[enc]()
    bs, nb = G.PACKED[enc][0], G.PACKED[enc][1]
    n, nblocks = 70, 4
    k = nblocks * bs
    blocks = G.weight_blocks(enc, n, nblocks, 0x5EED0020)
    x = G.floats(k, 0x5EED0021)
    want = L.gemv(enc, x, G.row_major(blocks), n)
    pad_x, pad_w, pad_y = 5, 2 * nb, 3
    xin = np.concatenate([np.full(pad_x, 9, np.float32), x])
    wbm = np.concatenate([np.full(pad_w, 0xAB, np.uint8), G.block_major(blocks)])
    out = np.full(pad_y + n + 2, 7, np.float32)
    kernel.matmul(xin, pad_x, wbm, pad_w, k, n, out, pad_y)
    assert (out[:pad_y] == 7).all() and (out[pad_y + n:] == 7).all()
    assert normalized_err(out[pad_y:pad_y + n], want) <= GEMV_TOL
    out2 = np.zeros(n, np.float32)
    kernel.matmul_row_major(x, 0, G.row_major(blocks), 0, k, n, out2, 0)
    assert np.array_equal(out2, out[pad_y:pad_y + n])
    with pytest.raises(ValueError):
        kernel.matmul(x, 0, wbm, 0, k - 1, n, out, 0)


def _device_bytes(kernels, w):
    """The device copy of an uploaded weight, byte for byte."""
    from skainet_amd import _lib
    out = np.empty(w.nbytes, np.uint8)
    assert _lib.hip().skainet_hip_memcpy_d2h(out.ctypes.data, w.data_ptr, out.size) == 0
    return out


@pytest.mark.parametrize("chunk_mib,lanes", [(0, 4), (1, 1), (1, 3), (1, 8), (8, 4)])
def test_weight_upload_through_the_page_locked_chunks_is_byte_exact(hip_backend, torch_cuda, chunk_mib, lanes):
    """A pageable source is staged through page-locked chunks, two per lane (one filled while the other is on the bus),
    the lanes on host threads of their own: a weight of many chunks with a ragged last one, with fewer chunks than the
    lanes could take, a weight smaller than a chunk, the staging switched off, a page-locked source (one transfer),
    and the input-block-major order (permuted on the device) all leave the same bytes on the device."""
    rng = np.random.default_rng(77 + chunk_mib + lanes)
    try:
        hip_backend.set_tuning("upload_chunk_mib", chunk_mib)
        hip_backend.set_tuning("upload_lanes", lanes)
        for enc, rows, cols in (("Q4_K", 4100, 4096), ("Q8_0", 37, 96), ("Q6_K", 3000, 2304)):
            bs, nb = G.PACKED[enc][0], G.PACKED[enc][1]
            per_row = cols // bs
            packed = rng.integers(0, 256, rows * per_row * nb, dtype=np.uint8)      # upload never interprets the bytes
            w = hip_backend.DeviceWeight.upload(enc, packed, rows, cols)
            assert np.array_equal(_device_bytes(hip_backend, w), packed), (enc, "pageable")
            w.close()
            pinned = hip_backend.PinnedBytes(packed.size)
            pinned.array[:] = packed
            w = hip_backend.DeviceWeight.upload(enc, pinned.array, rows, cols)
            assert np.array_equal(_device_bytes(hip_backend, w), packed), (enc, "page-locked")
            w.close()
            pinned.close()
            block_major = np.ascontiguousarray(packed.reshape(rows, per_row, nb).transpose(1, 0, 2)).reshape(-1)
            w = hip_backend.DeviceWeight.upload(enc, block_major, rows, cols, order=1)
            assert np.array_equal(_device_bytes(hip_backend, w), packed), (enc, "block-major")
            w.close()
    finally:
        hip_backend.set_tuning("upload_chunk_mib", 8)
        hip_backend.set_tuning("upload_lanes", 4)


@pytest.mark.parametrize("n,k", [(64, 4096), (37, 1024), (300, 8192)])
def test_q4k_one_row_fixed_point_kernel_at_the_extremes_of_its_digit_sums(hip_backend, torch_cuda, n, k):
    """Constant activations against saturated codes (all 15, all 0) with the largest scales: the top digit plane's sum
    passes 2^31 before the code sum takes its offset out again, so the recombination must be modular; and the negative
    mirror. Against the exact-fp32 oracle."""
    blocks = random_valid_blocks("Q4_K", n * k // 256, 11).reshape(n, k // 256, 144).copy()
    blocks[0::2, :, 16:] = 0xFF
    blocks[1::2, :, 16:] = 0x00
    blocks[:, :, 4:16] = 0xFF                                     # every 6-bit scale and minimum at 63
    packed = blocks.reshape(-1)
    for c in (7.5, -7.5, 1e-3):
        x = np.full((1, k), c, np.float32)
        got = gpu_matmul(hip_backend, torch_cuda, "Q4_K", packed, n, k, x)
        assert hip_backend.last_kernel() == "q4k_gemv_mfma_kernel"
        assert normalized_err(got, L.gemv("Q4_K", x, packed, n)) <= GEMV_TOL


def test_q4k_one_row_fixed_point_kernel_keeps_non_finite_activations_loud(hip_backend, torch_cuda):
    """The exact-fp32 product (ScalarQ4_KMatmulKernel.kt:40-78) propagates a NaN or an infinity among the activations into
    every output. The fixed-point kernel takes a group's largest magnitude with fmax (which drops a NaN) and scales by
    its reciprocal (0 for an infinity) -- but the sub-block's fp32 activation sum, which the minima multiply, carries
    the NaN or turns inf * 0 into one: no output stays finite. A group of subnormal activations contributes next to
    nothing, as in fp32. With the RMSNorm prologue the sum of squares does the same."""
    n, k = 64, 2048
    packed = random_valid_blocks("Q4_K", n * k // 256, 7)
    rng = np.random.default_rng(8)
    for bad in (np.nan, np.inf, -np.inf):
        x = rng.standard_normal((1, k)).astype(np.float32)
        x[0, 700] = bad
        got = gpu_matmul(hip_backend, torch_cuda, "Q4_K", packed, n, k, x)
        assert hip_backend.last_kernel() == "q4k_gemv_mfma_kernel"
        assert not np.isfinite(got).any(), bad
    x = rng.standard_normal((1, k)).astype(np.float32)
    x[0, 128:192] = np.float32(1e-41) * rng.standard_normal(64).astype(np.float32)      # one group of subnormals
    got = gpu_matmul(hip_backend, torch_cuda, "Q4_K", packed, n, k, x)
    assert np.isfinite(got).all() and normalized_err(got, L.gemv("Q4_K", x, packed, n)) <= GEMV_TOL
