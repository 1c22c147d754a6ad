"""The allocation-free form of the Lloyd update step (f2cgt_kmeans_update_static: partial sums in a
device array inside the library) against the workspace form, through the C ABI: two calls in a row,
the second on a smaller problem, so that what the first call left in the shared array must not show.
The sums are fp32 atomic adds in hardware order in both forms, hence the tolerance (rtol 1e-5 of the
data's scale, the bar of the aggregation results); untouched centres must agree bit for bit."""
import ctypes

import numpy as np
import pytest
import torch

from f2cgt_amd import capi

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def run_pair(lib, rng, m, n, k, u8):
    x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).cuda()
    start = torch.from_numpy(rng.standard_normal((n, k)).astype(np.float32)).cuda()
    labels = torch.from_numpy(rng.integers(0, max(1, n - 3), size=m)).cuda()      # the last clusters stay empty
    if u8:
        labels = labels.to(torch.uint8)
    stream = torch.cuda.current_stream().cuda_stream
    l64 = None if u8 else labels.data_ptr()
    l8 = labels.data_ptr() if u8 else None
    # the existing entry point, with a caller-allocated workspace
    want_c, want_s = start.clone(), torch.empty(2, device="cuda")
    ws = torch.empty((lib.f2cgt_kmeans_update_workspace_bytes(n, k),), dtype=torch.uint8, device="cuda")
    rc = lib.f2cgt_kmeans_update(x.data_ptr(), l64, l8, want_c.data_ptr(), want_s.data_ptr(), None, 0, 0.0,
                                 ws.data_ptr(), ws.numel(), m, n, k, stream)
    assert rc == 0, lib.f2cgt_last_error()
    # the allocation-free one: inputs and outputs only
    got_c, got_s = start.clone(), torch.empty(2, device="cuda")
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = lib.f2cgt_kmeans_update_static(x.data_ptr(), l64, l8, got_c.data_ptr(), got_s.data_ptr(), None, 0, 0.0,
                                        m, n, k, stream)
    assert rc == 0, lib.f2cgt_last_error()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    scale = float(x.abs().max())
    assert torch.allclose(got_c, want_c, rtol=RTOL, atol=RTOL * scale)
    if n > 3:
        assert torch.equal(got_c[n - 3:], start[n - 3:]) and torch.equal(want_c[n - 3:], start[n - 3:])
    assert torch.allclose(got_s, want_s, rtol=1e-4)
    return got_c


def test_static_scratch_matches_the_workspace_form_on_two_calls_in_a_row():
    lib = capi.lib()
    rng = np.random.default_rng(123)
    print("case kmeans_update_static 90000 x 32, 256 centres, then 7000 x 8, 12 centres", flush=True)
    run_pair(lib, rng, 90_000, 256, 32, True)
    run_pair(lib, rng, 7_000, 12, 8, False)      # smaller: most of the array still holds the first call's sums
    run_pair(lib, rng, 30_000, 1024, 64, False)  # exactly the largest sum table (65536 entries)


def test_static_scratch_rejects_what_does_not_fit():
    lib = capi.lib()
    a = ctypes.c_void_p(256)
    assert lib.f2cgt_kmeans_update_static(a, a, None, a, a, None, 0, 0.0, 10, 1024, 65, None) == -2
    assert b"65536" in lib.f2cgt_last_error()
    assert lib.f2cgt_kmeans_update_static(a, a, None, a, a, None, 0, 0.0, 10, 4097, 1, None) == -2
    assert lib.f2cgt_kmeans_update_static(a, a, a, a, a, None, 0, 0.0, 10, 16, 4, None) == -1    # both label kinds
