"""GPU radix sort and k-NN against library routines / brute force."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def H():
    import gpu_harness
    assert torch.cuda.is_available()
    return gpu_harness


@pytest.mark.parametrize("n", [1, 2, 63, 64, 65, 255, 2047, 2048, 2049, 100_003, 1_500_000])
@pytest.mark.parametrize("end_bit", [44, 45, 64, 33, 40])
def test_sort_pairs_u64(H, n, end_bit):
    rng = np.random.default_rng(n * 131 + end_bit)
    tile_bits = max(1, end_bit - 32)
    # few distinct depths per tile so ties exercise stability
    tiles = rng.integers(0, 1 << min(tile_bits, 12), n, dtype=np.uint64)
    depth = rng.integers(0, 50, n, dtype=np.uint64) * np.uint64(0x01010101)
    keys = (tiles << np.uint64(32)) | depth
    if end_bit < 64:
        # garbage above end_bit must be ignored by the comparison and carried along unchanged
        keys |= rng.integers(0, 2, n, dtype=np.uint64) << np.uint64(min(63, end_bit + 3))
    vals = np.arange(n, dtype=np.uint32)
    ko, vo = H.sort_pairs_u64(H.as_u64(keys), H.as_u32(vals), end_bit)
    mask = np.uint64((1 << end_bit) - 1) if end_bit < 64 else np.uint64(0xFFFFFFFFFFFFFFFF)
    order = np.argsort(keys & mask, kind="stable")
    assert np.array_equal(H.np_u32(vo), vals[order])
    assert np.array_equal(H.np_u64(ko), keys[order])


@pytest.mark.parametrize("n", [1, 1000, 2048, 4097, 777_777])
def test_sort_pairs_u32(H, n):
    rng = np.random.default_rng(n)
    keys = rng.integers(0, 1 << 30, n, dtype=np.uint32)
    keys[rng.integers(0, n, n // 3)] = keys[0]
    vals = rng.permutation(n).astype(np.uint32)
    ko, vo = H.sort_pairs_u32(H.as_u32(keys), H.as_u32(vals))
    order = np.argsort(keys, kind="stable")
    assert np.array_equal(H.np_u32(ko), keys[order])
    assert np.array_equal(H.np_u32(vo), vals[order])


@pytest.mark.parametrize("n", [1, 5, 2047, 2048, 2049, 1_000_001])
def test_inclusive_sum(H, n):
    rng = np.random.default_rng(n)
    x = rng.integers(0, 9, n, dtype=np.uint32)
    out = torch.empty(n, dtype=torch.int32, device=H.DEV)
    nb = H.lib.gs_scan_workspace_bytes(n)
    ws = torch.empty(nb, dtype=torch.uint8, device=H.DEV)
    xin = H.as_u32(x)
    H.gn.check(H.lib.gs_inclusive_sum(n, H.ptr(xin), H.ptr(out), H.ptr(ws), nb, H.stream()), "scan")
    torch.cuda.synchronize()
    assert np.array_equal(H.np_u32(out), np.cumsum(x, dtype=np.uint64).astype(np.uint32))


def _brute(points):
    from scipy.spatial import cKDTree
    d, _ = cKDTree(points.astype(np.float64)).query(points.astype(np.float64), k=4)
    return (d[:, 1:] ** 2).mean(axis=1)


@pytest.mark.parametrize("P,kind", [(7, "uniform"), (1024, "uniform"), (1025, "uniform"), (20_000, "uniform"),
                                    (20_000, "positive"), (50_000, "clustered"), (300_000, "slab")])
def test_knn_dist2(H, orc, P, kind):
    import simple_knn._C as knn
    rng = np.random.default_rng(P)
    if kind == "uniform":
        pts = rng.uniform(-10, 10, (P, 3))
    elif kind == "positive":
        pts = rng.uniform(5, 25, (P, 3))  # the zero-initialised bounding box reduction matters here
    elif kind == "clustered":
        pts = rng.normal(0, 1, (P, 3)) + rng.integers(0, 4, (P, 1)) * 30.0
    else:
        pts = rng.uniform(0, 1, (P, 3)) * np.array([200.0, 200.0, 30.0]) - np.array([100.0, 100.0, 0.0])
    pts = pts.astype(np.float32)
    got = knn.distCUDA2(torch.from_numpy(pts).to(H.DEV)).cpu().numpy()
    ref = orc.knn_dist2(pts)
    assert np.array_equal(got, ref), f"max abs diff {np.abs(got - ref).max()}"
    if P <= 50_000:
        np.testing.assert_allclose(got, _brute(pts), rtol=2e-4, atol=1e-9)


def _brute_f32(pts):
    """The three smallest squared distances of every point in float32 with the kernel's association,
    ((dx*dx + dy*dy) + dz*dz), and their mean ((a + b) + c) / 3: what any exact search must return, bit for bit.
    Distances that are not finite count as FLT_MAX, which is also what three missing neighbours read as."""
    big = np.float32(np.finfo(np.float32).max)
    out = np.empty(len(pts), np.float32)
    with np.errstate(all="ignore"):
        for i, p in enumerate(pts):
            d = pts - p
            d2 = (d[:, 0] * d[:, 0] + d[:, 1] * d[:, 1]) + d[:, 2] * d[:, 2]
            d2 = np.where(np.isnan(d2), big, np.minimum(d2, big)).astype(np.float32)
            d2[i] = big
            k = np.sort(np.concatenate([d2, np.full(3, big, np.float32)]))[:3]
            out[i] = ((k[0] + k[1]) + k[2]) / np.float32(3.0)
    return out


@pytest.mark.parametrize("case", ["one", "two", "three", "four", "63", "64", "65", "129", "identical", "duplicates",
                                  "line", "plane", "nan_and_inf", "far_outliers", "two_clusters", "2500"])
def test_knn_edge_cases_match_a_float32_brute_force(H, orc, case):
    import simple_knn._C as knn
    rng = np.random.default_rng(len(case) * 7 + ord(case[0]))
    n = {"one": 1, "two": 2, "three": 3, "four": 4}.get(case, int(case) if case.isdigit() else 1500)
    pts = rng.uniform(-5, 5, (n, 3)).astype(np.float32)
    if case == "identical":
        pts[:] = pts[0]
    elif case == "duplicates":
        pts = pts[rng.integers(0, 40, n)]
    elif case == "line":
        pts[:, 1:] = 0.25
    elif case == "plane":
        pts[:, 2] = -3.0
    elif case == "nan_and_inf":
        pts[rng.integers(0, n, 20), rng.integers(0, 3, 20)] = np.nan
        pts[rng.integers(0, n, 10), rng.integers(0, 3, 10)] = np.inf
        pts[rng.integers(0, n, 10), rng.integers(0, 3, 10)] = -np.inf
    elif case == "far_outliers":
        pts[::97] *= 1.0e6
    elif case == "two_clusters":
        pts[: n // 2] = pts[: n // 2] * 1e-3 + 1.0e4
    got = knn.distCUDA2(torch.from_numpy(pts).to(H.DEV)).cpu().numpy()
    want = _brute_f32(pts)
    assert np.array_equal(got, want, equal_nan=True), np.nonzero(got != want)[0][:10]
    if case not in ("nan_and_inf",):  # (the CPU statement's grid is undefined for non-finite bounds)
        assert np.array_equal(got, orc.knn_dist2(pts))


def test_cross_lane_reductions(H):
    rng = np.random.default_rng(0)
    x = rng.integers(-8, 9, (64, 16)).astype(np.float32)  # small integers: sums are exact in any order
    tin = H.dev(x)
    ow = torch.zeros(16, device=H.DEV)
    orow = torch.zeros(4, 16, device=H.DEV)
    H.gn.check(H.lib.gs_selftest_reductions(H.ptr(tin), H.ptr(ow), H.ptr(orow), H.stream()), "selftest")
    assert np.array_equal(ow.cpu().numpy(), x.sum(0))
    assert np.array_equal(orow.cpu().numpy(), x.reshape(4, 16, 16).sum(1))


def test_a_sort_that_gave_up_fails_the_next_call(H):
    """The radix sort's bounded wait is never made to run out on the GPU; instead the error word it would leave in
    its workspace is written by hand, and the plumbing behind it is followed: gs_sort_status reports it, the check
    kernel raises the sticky fault word without any wait, gs_pending_fault / the next composite call fail once and
    lower it, and the call after that works again."""
    from simple_knn._C import distCUDA2
    n = 10_000
    rng = np.random.default_rng(3)
    keys = rng.integers(0, 1 << 30, n, dtype=np.uint32)
    kin, vin = H.as_u32(keys), H.as_u32(np.arange(n, dtype=np.uint32))
    kout, vout = torch.empty_like(kin), torch.empty_like(vin)
    nb = H.lib.gs_sort_workspace_bytes(n)
    ws = torch.empty(nb, dtype=torch.uint8, device=H.DEV)
    H.gn.check(H.lib.gs_sort_pairs_u32(n, H.ptr(kin), H.ptr(kout), H.ptr(vin), H.ptr(vout), 32, H.ptr(ws), nb,
                                       H.stream()), "gs_sort_pairs_u32")
    assert H.lib.gs_sort_status(H.ptr(ws), H.stream()) == 0
    H.gn.check(H.lib.gs_sort_check_async(H.ptr(ws), H.stream()), "gs_sort_check_async")
    torch.cuda.synchronize()
    assert H.lib.gs_pending_fault() == 0
    # what a sort that gave up leaves behind
    base = (ws.data_ptr() + 255) // 256 * 256 - ws.data_ptr()
    off = base + H.lib.gs_sort_workspace_error_offset()
    ws[off:off + 4].view(torch.int32).fill_(1)
    assert H.lib.gs_sort_status(H.ptr(ws), H.stream()) == 1 and "not sorted" in H.gn.last_error()
    H.gn.check(H.lib.gs_sort_check_async(H.ptr(ws), H.stream()), "gs_sort_check_async")
    torch.cuda.synchronize()
    pts = torch.rand(1000, 3, device=H.DEV)
    with pytest.raises(RuntimeError, match="radix sort"):
        distCUDA2(pts)
    assert H.lib.gs_pending_fault() == 0  # lowered by the call that reported it
    assert distCUDA2(pts).shape == (1000,)
    # raised again: gs_pending_fault itself reports and lowers it
    H.gn.check(H.lib.gs_sort_check_async(H.ptr(ws), H.stream()), "gs_sort_check_async")
    torch.cuda.synchronize()
    assert H.lib.gs_pending_fault() == 1 and "radix sort" in H.gn.last_error()
    assert H.lib.gs_pending_fault() == 0
