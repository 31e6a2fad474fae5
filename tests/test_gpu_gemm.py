"""GPU parity: the MFMA dequant-GEMM (prefill) against the exact-fp32 oracle.

Tolerance stated by the task for the bf16-MFMA path: max relative error 2e-2 against the fp32 reference, measured
as |got - ref| / max(|ref|, 1e-2 * ||ref||_inf). The reference has no packed GEMM (m rows = m scalar GEMV calls,
PackedViewMatmulKernel.kt:99), which is exactly what the oracle does here.
"""
import numpy as np
import pytest

from oracle import golden as G
from oracle import lib as L
from gpu_util import ENCS, MORE_ENCS, dev, gaussian_weight, normalized_err, random_valid_blocks

ALL_ENCS = ENCS + MORE_ENCS

pytestmark = pytest.mark.gpu
GEMM_TOL = 2e-2       # max |got - ref| / ||ref||_inf against the exact-fp32 oracle
GEMM_RMS_TOL = 1e-2   # RMS(err) / RMS(ref), the aggregate form the reference uses for its own reduced-precision path
                      # (NativeQ4KMatmulKernelParityTest.kt:84-103, bound 0.03 there)
EXACT_TOL = 2e-4      # against the same product with both operands rounded to bf16 first (what the kernel computes)


def check(got, want_fp32):
    """bf16-MFMA bound: operands carry 8 significant bits, so an output near zero has an unbounded per-element
    relative error; the bound is taken against the largest output (and in aggregate)."""
    err = normalized_err(got, want_fp32, eps=1.0)
    rms = float(np.sqrt(((got - want_fp32.astype(np.float64)) ** 2).mean()) / max(np.sqrt((want_fp32.astype(np.float64) ** 2).mean()), 1e-30))
    assert err <= GEMM_TOL and rms <= GEMM_RMS_TOL, (err, rms)
    return err


def bf16_round(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a, np.float32)).to(torch.bfloat16).to(torch.float64).numpy()


def check_exact(torch, enc, got, x, packed, n):
    """The kernel's own arithmetic restated: decode (oracle, fp32) -> bf16, activations -> bf16, exact products, wide sums.
    Only the fp32 accumulation order is left, so a wrong fragment layout or a misplaced scale cannot hide."""
    w = bf16_round(torch, L.dequant(enc, packed).reshape(n, -1))
    want = bf16_round(torch, x) @ w.T
    assert normalized_err(got, want) <= EXACT_TOL, normalized_err(got, want)


def gpu_gemm(kernels, torch, enc, packed, n, k, x, kind=1):
    w = kernels.DeviceWeight.upload(enc, packed, n, k)
    m = x.shape[0]
    y = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
    w.matmul(dev(torch, x), m, y, kind)
    return y.cpu().numpy()


@pytest.mark.parametrize("enc", ALL_ENCS)
@pytest.mark.parametrize("m,n,k", [(9, 5, 256), (33, 130, 512), (256, 128, 1024), (300, 257, 768), (64, 1000, 2304), (1, 64, 256)])
def test_gemm_ragged_tiles(hip_backend, torch_cuda, enc, m, n, k):
    packed = gaussian_weight(hip_backend, enc, n, k, 200 + n)
    x = np.random.default_rng(m + k).standard_normal((m, k)).astype(np.float32)
    got = gpu_gemm(hip_backend, torch_cuda, enc, packed, n, k, x)
    want = L.gemv(enc, x, packed, n)
    assert not np.isnan(got).any()
    check(got, want)
    check_exact(torch_cuda, enc, got, x, packed, n)
    # the automatic choice (m > 8 -> GEMM, else GEMV) gives the same product
    auto = gpu_gemm(hip_backend, torch_cuda, enc, packed, n, k, x, kind=None)
    check(auto, want)
    # and so does the wide (256 x 256) tile, which the launcher would only pick for weights of many rows
    try:
        hip_backend.set_tuning("gemm_wide", 1)
        wide = gpu_gemm(hip_backend, torch_cuda, enc, packed, n, k, x)
        assert not np.isnan(wide).any()
        check(wide, want)
        check_exact(torch_cuda, enc, wide, x, packed, n)
    finally:
        hip_backend.set_tuning("gemm_wide", -1)


@pytest.mark.parametrize("enc", ALL_ENCS)
def test_gemm_on_random_valid_blocks_and_forced_k_splits(hip_backend, torch_cuda, enc):
    bs = G.PACKED[enc][0]
    m, n, k = 40, 200, 2048
    packed = random_valid_blocks(enc, n * k // bs, 300)
    x = np.random.default_rng(5).standard_normal((m, k)).astype(np.float32)
    want = L.gemv(enc, x, packed, n)
    try:
        for rows in (2, 4):                      # 128 / 256 activation rows per tile (40 rows would pick 128 by itself)
            hip_backend.set_tuning("gemm_rows", rows)
            for wide in (0, 1):
                hip_backend.set_tuning("gemm_wide", wide)
                for ks in (1, 2, 3, 8):
                    hip_backend.set_tuning("gemm_ksplit", ks)
                    got = gpu_gemm(hip_backend, torch_cuda, enc, packed, n, k, x)
                    check(got, want)
                    check_exact(torch_cuda, enc, got, x, packed, n)
    finally:
        hip_backend.set_tuning("gemm_ksplit", 0)
        hip_backend.set_tuning("gemm_wide", -1)
        hip_backend.set_tuning("gemm_rows", 0)


@pytest.mark.parametrize("k", [96, 192, 320, 448])
def test_gemm_q8_0_rows_that_are_not_whole_256_element_groups_fall_back_to_the_row_kernels(hip_backend, torch_cuda, k):
    """The tile kernel's K loop runs over whole 256-element groups; a Q8_0 row of 3, 6, 10 or 14 blocks takes the
    row kernels instead (exact fp32 products, so the one-row bound applies)."""
    m, n = 20, 50
    packed = gaussian_weight(hip_backend, "Q8_0", n, k, 7)
    x = np.random.default_rng(8).standard_normal((m, k)).astype(np.float32)
    got = gpu_gemm(hip_backend, torch_cuda, "Q8_0", packed, n, k, x)
    assert normalized_err(got, L.gemv("Q8_0", x, packed, n)) <= 1e-3


@pytest.mark.parametrize("enc,n,k", [("Q4_K", 4096, 4096), ("Q6_K", 32000, 4096), ("Q4_K", 14336, 4096), ("Q4_K", 4096, 14336)])
def test_gemm_at_config_sizes(hip_backend, torch_cuda, enc, n, k):
    """Prefill configuration: activations 512 x 4096 ~ N(0, 1). The oracle checks 6 sampled activation rows in full
    (each a scalar GEMV over the whole weight); linearity ties the rest of the batch to those rows."""
    m = 512
    packed = gaussian_weight(hip_backend, enc, n, k, 400)
    rng = np.random.default_rng(401)
    x = rng.standard_normal((m, k)).astype(np.float32)
    got = gpu_gemm(hip_backend, torch_cuda, enc, packed, n, k, x)
    rows = [0, 1, 255, 256, 300, 511]
    want = L.gemv(enc, x[rows], packed, n)
    err = check(got[rows], want)
    print(f"{enc} {m}x{n}x{k}: normalized max err {err:.2e}")
    check_exact(torch_cuda, enc, got[rows], x[rows], packed, n)
    # size-independent property over the whole batch: C is linear in A -- (P A) W^T == P (A W^T) for a mixing matrix P
    p = rng.standard_normal((8, m)).astype(np.float32) / np.sqrt(m)
    mixed = gpu_gemm(hip_backend, torch_cuda, enc, packed, n, k, (p.astype(np.float64) @ x).astype(np.float32))
    check(mixed, (p.astype(np.float64) @ got).astype(np.float32))
    # and the GEMM agrees with the fp32 row kernels on the same device
    few = gpu_gemm(hip_backend, torch_cuda, enc, packed, n, k, x[:4].copy(), kind=0)
    check(got[:4], few)


@pytest.mark.parametrize("m,n,k", [(512, 4096, 4096), (9, 64, 256), (130, 70, 512), (128, 129, 1024), (300, 1000, 2304), (40, 200, 14336),
                                   (257, 63, 768)])
def test_q4k_gemm_with_k_split_over_the_waves(hip_backend, torch_cuda, m, n, k):
    """The Q4_K kernel that gives every wave the whole 128 x 64 tile and a share of K, forced on shapes with ragged row
    and column tiles, one and many super-blocks per row, and the shape the launcher picks it for by itself; against the
    oracle (2e-2) and against the same product with both operands rounded to bf16 first (2e-4)."""
    packed = gaussian_weight(hip_backend, "Q4_K", n, k, 900 + n)
    x = np.random.default_rng(m * 7 + k).standard_normal((m, k)).astype(np.float32)
    want = L.gemv("Q4_K", x, packed, n)
    try:
        hip_backend.set_tuning("gemm_ksw", 2)
        got = gpu_gemm(hip_backend, torch_cuda, "Q4_K", packed, n, k, x)
        assert hip_backend.last_kernel() == "q4k_gemm_ksw_kernel"
        assert not np.isnan(got).any()
        check(got, want)
        check_exact(torch_cuda, "Q4_K", got, x, packed, n)
        # one team of four waves per workgroup instead of two (each team takes half of K where the super-blocks split
        # evenly), with the fewest and the most activation stages in LDS: same operands, another fp32 summation order
        for stages in (3, 7):
            hip_backend.set_tuning("gemm_ksw_teams", 1)
            hip_backend.set_tuning("gemm_ksw_stages", stages)
            one_team = gpu_gemm(hip_backend, torch_cuda, "Q4_K", packed, n, k, x)
            assert hip_backend.last_kernel() == "q4k_gemm_ksw_kernel"
            assert normalized_err(got, one_team) <= 1e-4
        hip_backend.set_tuning("gemm_ksw", 0)
        tiles = gpu_gemm(hip_backend, torch_cuda, "Q4_K", packed, n, k, x)
        assert hip_backend.last_kernel() == "dequant_gemm_kernel"
        assert normalized_err(got, tiles) <= 1e-4          # same operands, another fp32 summation order
    finally:
        hip_backend.set_tuning("gemm_ksw", 1)
        hip_backend.set_tuning("gemm_ksw_teams", 2)
        hip_backend.set_tuning("gemm_ksw_stages", 5)


@pytest.mark.parametrize("m,n,k", [(512, 4096, 4096), (9, 64, 256), (130, 70, 512), (128, 129, 1024), (300, 1000, 2304), (40, 200, 14336),
                                   (257, 63, 768), (64, 512, 11008), (384, 1024, 4096)])
def test_q4k_gemm_with_activations_in_fragment_order(hip_backend, torch_cuda, m, n, k):
    """The Q4_K kernel whose activations are laid out by the pass in front in the order the matrix instruction reads them
    (every wave: the whole 128 x 64 tile and whole super-blocks of K), in both of its forms (eight waves per workgroup,
    and four with two workgroups per CU), forced on shapes with ragged row and column tiles,
    fewer super-blocks than waves, uneven super-block counts per wave (43 and 56 super-blocks over 8 waves), tile counts
    that are and are not a multiple of the eight dies; against the oracle (2e-2), against the same product with both
    operands rounded to bf16 first (2e-4), and against the tile kernel."""
    packed = gaussian_weight(hip_backend, "Q4_K", n, k, 900 + n)
    x = np.random.default_rng(m * 7 + k).standard_normal((m, k)).astype(np.float32)
    want = L.gemv("Q4_K", x, packed, n)
    try:
        hip_backend.set_tuning("gemm_frag", 2)
        for waves in (8, 4):                       # one workgroup of eight waves per CU, or two of four
            hip_backend.set_tuning("gemm_frag_waves", waves)
            got = gpu_gemm(hip_backend, torch_cuda, "Q4_K", packed, n, k, x)
            assert hip_backend.last_kernel() == "q4k_gemm_frag_kernel"
            assert not np.isnan(got).any()
            check(got, want)
            check_exact(torch_cuda, "Q4_K", got, x, packed, n)
        hip_backend.set_tuning("gemm_frag", 0)
        hip_backend.set_tuning("gemm_ksw", 0)
        tiles = gpu_gemm(hip_backend, torch_cuda, "Q4_K", packed, n, k, x)
        assert hip_backend.last_kernel() == "dequant_gemm_kernel"
        assert normalized_err(got, tiles) <= 1e-4          # same operands, another fp32 summation order
    finally:
        hip_backend.set_tuning("gemm_frag", 1)
        hip_backend.set_tuning("gemm_frag_waves", 0)
        hip_backend.set_tuning("gemm_ksw", 1)
    if (m, n, k) == (512, 4096, 4096):
        gpu_gemm(hip_backend, torch_cuda, "Q4_K", packed, n, k, x)
        assert hip_backend.last_kernel() == "q4k_gemm_frag_kernel"     # the launcher's own choice for this shape
