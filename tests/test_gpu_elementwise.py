"""Device elementwise, activation and reduction entries against float64 closed forms and, where the reference's C library
was built from its sources (oracle/_ref), against that library on the same inputs. Add / sub / mul / div are IEEE
operations: bit-exact against numpy, and against the reference library except its quotients (built with -ffast-math, it
multiplies by a reciprocal: one unit in the last place). Activations use the device's expf / tanhf / erf: 2e-6 of max(1, |ref|). Sums differ from a
sequential float sum by rounding order only: 1e-5 of the sum of magnitudes."""
import ctypes as C

import numpy as np
import pytest

from oracle import lib as L
from gpu_util import dev

pytestmark = pytest.mark.gpu


def _ref_lib():
    ref = L.ref()
    if ref is None or not hasattr(ref, "skainet_f32_binary"):
        return None
    fp = C.POINTER(C.c_float)
    ref.skainet_f32_binary.argtypes = [C.c_int32, fp, C.c_int32, fp, C.c_int32, fp, C.c_int32, C.c_int32]
    ref.skainet_f32_binary.restype = None
    ref.skainet_f32_unary.argtypes = [C.c_int32, fp, fp, C.c_int32]
    ref.skainet_f32_unary.restype = None
    ref.skainet_f32_reduce_all.argtypes = [fp, C.c_int32, C.c_int32, fp]
    ref.skainet_f32_reduce_all.restype = None
    ref.skainet_f32_reduce_axis.argtypes = [fp, C.c_int32, C.c_int32, C.c_int32, C.c_int32, fp]
    ref.skainet_f32_reduce_axis.restype = None
    return ref


@pytest.mark.parametrize("n,inner", [(1, 1), (1000, 8), (4096, 4096), (12345, 15), (1 << 20, 1024)])
def test_binary_ops_and_operand_modes(hip_backend, torch_cuda, n, inner):
    torch, kx = torch_cuda, hip_backend
    rng = np.random.default_rng(n)
    ref = _ref_lib()
    full_a = rng.standard_normal(n).astype(np.float32)
    full_b = (rng.standard_normal(n) + 3.0).astype(np.float32)          # away from zero for the quotients
    for op, f in (("add", np.add), ("sub", np.subtract), ("mul", np.multiply), ("div", np.divide)):
        for a_mode, b_mode in ((0, 0), (0, 1), (0, 2), (1, 0), (2, 0), (2, 2), (1, 2)):
            size = {0: n, 1: 1, 2: inner}
            a, b = full_a[:size[a_mode]].copy(), full_b[:size[b_mode]].copy()
            idx = np.arange(n)
            ia = idx if a_mode == 0 else (np.zeros(n, np.int64) if a_mode == 1 else idx % inner)
            ib = idx if b_mode == 0 else (np.zeros(n, np.int64) if b_mode == 1 else idx % inner)
            want = f(a[ia], b[ib]).astype(np.float32)
            out = torch.full((n + 3,), 7.0, dtype=torch.float32, device="cuda")
            kx.binary_dev(op, dev(torch, a), dev(torch, b), out, n, a_mode, b_mode, inner)
            kx.sync()
            got = out.cpu().numpy()
            assert np.array_equal(got[:n].view(np.uint32), want.view(np.uint32)), (op, a_mode, b_mode)
            assert (got[n:] == 7.0).all()
            if ref is not None and n <= 12345:
                r = np.empty(n, np.float32)
                ref.skainet_f32_binary(kx.BINARY_OPS[op], L.fp(a), a_mode, L.fp(b), b_mode, L.fp(r), n, inner)
                if op == "div":      # the reference builds with -ffast-math: a scalar divisor becomes a reciprocal multiply
                    assert (np.abs(got[:n] - r) <= 1.2e-7 * np.abs(r)).all(), (op, a_mode, b_mode)
                else:
                    assert np.array_equal(got[:n].view(np.uint32), r.view(np.uint32)), (op, a_mode, b_mode)
    from skainet_amd._lib import HipError
    with pytest.raises(HipError):
        kx.binary_dev("add", out, out, out, 4, 3, 0, 1)                 # unknown operand mode
    kx.binary_dev("add", out, out, out, 0)                              # nothing to do is not an error


def test_unary_activations(hip_backend, torch_cuda):
    import math
    torch, kx = torch_cuda, hip_backend
    rng = np.random.default_rng(5)
    x = np.concatenate([rng.standard_normal(100000) * 3.0, [0.0, -0.0, 20.0, -20.0, 88.0, -88.0, 1e-8, -1e-8]]).astype(np.float32)
    n = x.size
    x64 = x.astype(np.float64)
    erf = np.vectorize(math.erf)
    closed = {
        "relu": np.where(x64 < 0, 0.0, x64),
        "sigmoid": 1.0 / (1.0 + np.exp(-x64)),
        "silu": x64 / (1.0 + np.exp(-x64)),
        "gelu_tanh": 0.5 * x64 * (1.0 + np.tanh(np.float64(np.float32(0.7978845608)) * (x64 + np.float64(np.float32(0.044715)) * x64 ** 3))),
        "gelu": 0.5 * x64 * (1.0 + erf(x64 * 0.70710678118654752440)),
        "erf": erf(x64),
        "tanh": np.tanh(x64),
    }
    ref = _ref_lib()
    xd = dev(torch, x)
    for op, want in closed.items():
        out = torch.empty(n, dtype=torch.float32, device="cuda")
        kx.unary_dev(op, xd, out, n)
        kx.sync()
        got = out.cpu().numpy().astype(np.float64)
        err = np.abs(got - want) / np.maximum(1.0, np.abs(want))
        assert err.max() <= 2e-6, (op, err.max(), x[err.argmax()])
        if op == "relu":
            assert np.array_equal(out.cpu().numpy(), np.where(x < 0, np.float32(0), x))
        if ref is not None:
            r = np.empty(n, np.float32)
            ref.skainet_f32_unary(kx.UNARY_OPS[op], L.fp(x), L.fp(r), n)
            assert (np.abs(got - r) / np.maximum(1.0, np.abs(r))).max() <= 2e-6, op
    from skainet_amd._lib import HipError
    with pytest.raises(HipError):
        hip_backend.check(hip_backend._lib.hip().skainet_hip_f32_unary_dev(9, hip_backend._ptr(xd), hip_backend._ptr(xd), 4), "unary")


@pytest.mark.parametrize("n", [0, 1, 63, 4096, 100003, 1 << 22])
def test_reduce_all_sum_and_mean(hip_backend, torch_cuda, n):
    torch, kx = torch_cuda, hip_backend
    rng = np.random.default_rng(n + 1)
    x = (rng.standard_normal(max(n, 1)) + 0.25).astype(np.float32)
    xd = dev(torch, x)
    ref = _ref_lib()
    for mean in (False, True):
        out = torch.full((2,), 7.0, dtype=torch.float32, device="cuda")
        kx.reduce_all_dev(xd, n, out, mean)
        kx.sync()
        got = out.cpu().numpy()
        want = float(x[:n].astype(np.float64).sum()) / (n if (mean and n > 0) else 1)
        tol = 1e-5 * float(np.abs(x[:n]).astype(np.float64).sum()) / (n if (mean and n > 0) else 1) + 1e-30
        assert abs(float(got[0]) - want) <= tol, (n, mean, got[0], want)
        assert got[1] == 7.0
        if ref is not None and 0 < n <= 100003:
            r = np.zeros(1, np.float32)
            ref.skainet_f32_reduce_all(L.fp(x), n, int(mean), L.fp(r))
            assert abs(float(got[0]) - float(r[0])) <= 4 * tol


@pytest.mark.parametrize("outer,red,inner", [(1, 1, 1), (7, 13, 5), (4, 4096, 1), (3, 1000, 2), (32, 128, 128), (2, 3, 4096), (512, 4096, 1)])
def test_reduce_axis_sum_and_mean(hip_backend, torch_cuda, outer, red, inner):
    torch, kx = torch_cuda, hip_backend
    rng = np.random.default_rng(outer * red + inner)
    x = rng.standard_normal((outer, red, inner)).astype(np.float32)
    xd = dev(torch, x)
    ref = _ref_lib()
    for mean in (False, True):
        out = torch.full((outer * inner + 1,), 7.0, dtype=torch.float32, device="cuda")
        kx.reduce_axis_dev(xd, outer, red, inner, out, mean)
        kx.sync()
        got = out.cpu().numpy()
        want = x.astype(np.float64).sum(1) / (red if mean else 1)
        tol = 1e-5 * np.abs(x).astype(np.float64).sum(1) / (red if mean else 1) + 1e-30
        assert (np.abs(got[:-1].reshape(outer, inner) - want) <= tol).all()
        assert got[-1] == 7.0
        if ref is not None:
            r = np.empty(outer * inner, np.float32)
            ref.skainet_f32_reduce_axis(L.fp(x), outer, red, inner, int(mean), L.fp(r))
            assert (np.abs(got[:-1] - r).reshape(outer, inner) <= 4 * tol).all()
