"""The arg-max entry that allocates nothing (fixed scratch array inside the library) against the allocating entry it
mirrors: two calls in a row through the C ABI, the second on a smaller input, plus the refusal beyond its row limit."""
import numpy as np
import pytest

from skainet_amd import _lib
from tests.gpu_util import dev

pytestmark = pytest.mark.gpu


def test_argmax_noalloc_matches_the_allocating_entry(hip_backend, torch_cuda):
    torch, kx = torch_cuda, hip_backend
    lib = _lib.hip()
    for rows, cols, seed in ((5, 128256, 1), (2, 20000, 2)):          # the second call is the smaller one
        lg = np.random.default_rng(seed).standard_normal((rows, cols)).astype(np.float32)
        lg[0, cols - 1] = lg[0, cols // 3] = 40.0                     # a tie across two slices keeps the lower index
        lg[1, :] = -2.5                                               # all equal: index 0
        d = dev(torch, lg)
        want = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        got = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
        assert lib.skainet_hip_f32_argmax_rows_dev(d.data_ptr(), rows, cols, want.data_ptr()) == 0, _lib.last_error()
        assert lib.skainet_hip_f32_argmax_rows_noalloc_dev(d.data_ptr(), rows, cols, got.data_ptr()) == 0, _lib.last_error()
        kx.sync()
        assert got.cpu().tolist() == want.cpu().tolist() == [int(r.argmax()) for r in lg]   # integer output: exact
        assert got.cpu().tolist()[:2] == [cols // 3, 0]


def test_argmax_noalloc_refuses_more_rows_than_its_scratch_holds(hip_backend, torch_cuda):
    torch = torch_cuda
    lib = _lib.hip()
    x = torch.zeros((65, 32), device="cuda")
    out = torch.full((65,), -7, dtype=torch.int32, device="cuda")
    assert lib.skainet_hip_f32_argmax_rows_noalloc_dev(x.data_ptr(), 65, 32, out.data_ptr()) == -1
    assert "65 rows exceed" in _lib.last_error()
    hip_backend.sync()
    assert (out.cpu().numpy() == -7).all()                           # refused on the host: nothing ran
    # short rows are served too (the allocating entry would take its one-workgroup kernel here)
    y = dev(torch, np.arange(64 * 10, dtype=np.float32).reshape(64, 10) % 7)
    got = torch.empty(64, dtype=torch.int32, device="cuda")
    assert lib.skainet_hip_f32_argmax_rows_noalloc_dev(y.data_ptr(), 64, 10, got.data_ptr()) == 0
    hip_backend.sync()
    assert got.cpu().tolist() == [int(r.argmax()) for r in y.cpu().numpy()]


def test_argmax_noalloc_from_two_host_threads_at_once(hip_backend, torch_cuda):
    """Two host threads, each on its own stream (the library's streams are per thread), call the entry over and over on
    different inputs: each thread has a slot of the fixed array to itself, so no call sees the other's counters."""
    import threading
    torch = torch_cuda
    lib = _lib.hip()
    rng = np.random.default_rng(9)
    data = [rng.standard_normal((3, 50000)).astype(np.float32) for _ in range(2)]
    devs = [dev(torch, d) for d in data]
    outs = [torch.full((40, 3), -1, dtype=torch.int32, device="cuda") for _ in range(2)]
    errs = []

    def work(t):
        assert lib.skainet_hip_thread_stream() == 0, _lib.last_error()       # so that the two threads' kernels can overlap
        for i in range(40):
            if lib.skainet_hip_f32_argmax_rows_noalloc_dev(devs[t].data_ptr(), 3, 50000, outs[t][i].data_ptr()) != 0:
                errs.append(_lib.last_error())
        lib.skainet_hip_sync()
        lib.skainet_hip_thread_release()

    torch.cuda.synchronize()                                                 # the inputs are on the device before the threads start
    ts = [threading.Thread(target=work, args=(t,)) for t in range(2)]
    [t.start() for t in ts]
    [t.join() for t in ts]
    assert not errs, errs
    torch.cuda.synchronize()
    for t in range(2):
        want = [int(r.argmax()) for r in data[t]]
        assert (outs[t].cpu().numpy() == np.array(want, np.int32)).all()
