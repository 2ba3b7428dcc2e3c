"""The entry point that allocates nothing (gs_inclusive_sum_static) against gs_inclusive_sum, through the C ABI."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def H():
    import gpu_harness
    assert torch.cuda.is_available()
    return gpu_harness


def _both(H, x):
    n = x.shape[0]
    xin = H.as_u32(x)
    ref = torch.full((n,), -1, dtype=torch.int32, device=H.DEV)
    nb = H.lib.gs_scan_workspace_bytes(n)
    ws = torch.empty(nb, dtype=torch.uint8, device=H.DEV)
    H.gn.check(H.lib.gs_inclusive_sum(n, H.ptr(xin), H.ptr(ref), H.ptr(ws), nb, H.stream()), "gs_inclusive_sum")
    out = torch.full((n,), -2, dtype=torch.int32, device=H.DEV)
    torch.cuda.synchronize()
    # free device memory as the driver sees it (an allocation inside the library would not show in torch's own
    # counters), and torch's counters for the wrapper side
    free_before, before = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    H.gn.check(H.lib.gs_inclusive_sum_static(n, H.ptr(xin), H.ptr(out), H.stream()), "gs_inclusive_sum_static")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    return H.np_u32(ref), H.np_u32(out)


def test_static_scan_matches_workspace_scan_twice_in_a_row(H):
    rng = np.random.default_rng(7)
    # (the first call on a device looks the static array's address up; the calls measured below come after it)
    t0 = H.as_u32(np.array([1, 2, 3], np.uint32))
    H.gn.check(H.lib.gs_inclusive_sum_static(3, H.ptr(t0), H.ptr(t0), H.stream()), "gs_inclusive_sum_static")
    torch.cuda.synchronize()
    # two calls in a row on the same GPU (they share the static array), the second with a smaller input
    for n in (3_000_001, 70_003):
        x = rng.integers(0, 9, n, dtype=np.uint32)
        ref, out = _both(H, x)
        assert np.array_equal(out, ref)
        assert np.array_equal(out, np.cumsum(x, dtype=np.uint64).astype(np.uint32))
    # in place, a single element, and a sum that wraps around 2^32 like the workspace version's
    x = np.full(5000, 0x00200000, np.uint32)
    ref, out = _both(H, x)
    assert np.array_equal(out, ref)
    t = H.as_u32(np.array([5], np.uint32))
    H.gn.check(H.lib.gs_inclusive_sum_static(1, H.ptr(t), H.ptr(t), H.stream()), "gs_inclusive_sum_static")
    torch.cuda.synchronize()
    assert H.np_u32(t)[0] == 5


def test_static_scan_refuses_sizes_beyond_its_array(H):
    cap = H.lib.gs_inclusive_sum_static_max()
    assert cap == 1 << 27
    t = torch.zeros(16, dtype=torch.int32, device=H.DEV)
    assert H.lib.gs_inclusive_sum_static(cap + 1, H.ptr(t), H.ptr(t), H.stream()) != 0
    assert "exceeds" in H.gn.last_error() and "capacity" in H.gn.last_error()
    assert H.lib.gs_inclusive_sum_static(-1, H.ptr(t), H.ptr(t), H.stream()) != 0
    assert H.lib.gs_inclusive_sum_static(0, None, None, H.stream()) == 0
    # the refusal left the library usable
    x = np.arange(4096, dtype=np.uint32)
    ref, out = _both(H, x)
    assert np.array_equal(out, ref)
