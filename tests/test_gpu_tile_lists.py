"""The per-tile lists render_gaussians builds (ranges, sorted keys, point_list), by each of its routes: instances
bucketed by tile and sorted per tile (in registers, by the per-tile radix sort inside one CU, or by the per-tile radix
sort block by block through memory), and the radix sort over all (tile | depth) keys.  Every route must give the
oracle's lists bit for bit, and the backward pass must file its per-instance gradients correctly under each."""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def H():
    import gpu_harness
    return gpu_harness


def _mask(kind, gx, gy):
    cl = torch.ones(gy, gx, dtype=torch.bool)
    if kind == "rows":
        cl[: gy // 3] = False
    elif kind == "checker":
        yy, xx = torch.meshgrid(torch.arange(gy), torch.arange(gx), indexing="ij")
        cl = ((yy + xx) % 2 == 0)
    return cl


# (longest list sorted in registers, records the per-tile radix sort holds at once): defaults; lists of more than 40
# records by the per-tile radix sort's two kernels; the radix sort over all keys; lists of more than 40 records by
# the smaller kernel up to 64 and block by block beyond (blocks of 64, of 128, and many blocks of an odd size)
ROUTES = [(-1, -1), (40, 0), (0, 0), (40, 64), (100, 128), (7, 7)]


@pytest.mark.parametrize("cfg,P,mask", [(0, 30_000, "all"), (1, 120_000, "all"), (1, 60_000, "checker"),
                                        (3, 40_000, "rows")])
def test_lists_match_oracle_by_every_route(orc, H, cfg, P, mask):
    import gs_scenes
    import gsrast_native as gn
    from diff_gaussian_rasterization import _C
    g, cams = gs_scenes.make_scene(cfg, P=P, n_views=1)
    cam = cams[0]
    W, Hh = cam.image_width, cam.image_height
    gx, gy = H.grid(W, Hh)
    T = gx * gy
    cl = _mask(mask, gx, gy)
    o, gd = H.preprocess_fwd(g, cam)
    vm, cp = cam.world_view_transform.to(DEV), cam.camera_center.to(DEV)
    am = gs_scenes.build_all_map(gd["means3D"], gd["scales"], gd["rotations"], cam)
    n = lambda t: t.detach().cpu().numpy()
    want = orc.bin_and_sort(n(o["radii"]), n(o["means2D"]), n(o["depths"]), cl.numpy().reshape(-1), W, Hh)
    R_want = int(want["point_list"].shape[0])
    counts = want["ranges"].reshape(-1, 2).astype(np.int64)
    longest = int((counts[:, 1] - counts[:, 0]).max())
    assert longest > 64  # so that the blocked routes really sort lists of more than one block
    ug = gs_scenes.upstream_grads(cam)
    args = {"stats_collector": {}}
    grads = []
    for large, chunks in ROUTES:
        args["tile_sort_limits"] = (large, chunks)
        out = _C.render_gaussians(torch.zeros(3, device=DEV), Hh, W, o["means2D"], o["depths"], o["radii"],
                                  o["conic_opacity"], o["rgb"], cl.to(DEV), vm, cp, cam.tanfovx, cam.tanfovy, am,
                                  True, False, args)
        R, color, n_render, n_consider, n_contrib, out_observe, oam, opd, geomB, binB, imgB = out
        assert R == R_want
        off = [C.c_size_t() for _ in range(5)]
        gn.check(gn.lib.gs_binning_state_layout(R, W, Hh, *[C.byref(x) for x in off]), "layout")
        base = (binB.data_ptr() + 255) // 256 * 256 - binB.data_ptr()
        point_list = binB[base + off[0].value: base + off[0].value + 4 * R].view(torch.int32)
        keys = binB[base + off[1].value: base + off[1].value + 8 * R].view(torch.int64)
        ioff = [C.c_size_t() for _ in range(5)]
        gn.check(gn.lib.gs_image_state_layout(W, Hh, *[C.byref(x) for x in ioff]), "layout")
        ibase = (imgB.data_ptr() + 255) // 256 * 256 - imgB.data_ptr()
        ranges = imgB[ibase + ioff[3].value: ibase + ioff[3].value + 8 * T].view(torch.int32)
        assert np.array_equal(H.np_u32(ranges), want["ranges"].reshape(-1)), (large, chunks)
        assert np.array_equal(H.np_u32(point_list), want["point_list"]), (large, chunks)
        assert np.array_equal(H.np_u64(keys), want["keys"]), (large, chunks)
        assert np.array_equal(n(n_render), (counts[:, 1] - counts[:, 0]).astype(np.int32))
        back = _C.render_gaussians_backward(torch.zeros(3, device=DEV), cam.tanfovx, cam.tanfovy, oam, am, R, geomB,
                                            binB, imgB, cl.to(DEV), ug["color"].to(DEV), ug["all_map"].to(DEV),
                                            ug["plane_depth"].to(DEV), o["means2D"], o["conic_opacity"], o["rgb"],
                                            True, False, args)
        grads.append((color, [b.clone() for b in back]))
    # the lists are identical, so every route gives the same image bit for bit and the same gradients up to the
    # order of the LDS sums inside a tile
    # (pixels of tiles that are not computed locally are left untouched, so only the others are compared)
    px = cl.repeat_interleave(16, 0).repeat_interleave(16, 1)[:Hh, :W].to(DEV)
    for color, back in grads[1:]:
        assert torch.equal(color[:, px], grads[0][0][:, px])
        for a, b in zip(back, grads[0][1]):
            assert float((a - b).norm()) <= 1e-5 * float(b.norm()) + 1e-12
    f = orc.render_fwd(want["ranges"], want["point_list"], n(o["means2D"]), n(o["rgb"]), n(am), n(o["conic_opacity"]),
                       cl.numpy().reshape(-1), np.zeros(3, np.float32), W, Hh, cam.tanfovx, cam.tanfovy)
    rb = orc.render_bwd(want["ranges"], want["point_list"], n(o["means2D"]), n(o["conic_opacity"]), n(o["rgb"]), n(am),
                        f["out_all_map"], f["final_T"], f["n_contrib"], cl.numpy().reshape(-1), np.zeros(3, np.float32),
                        n(ug["color"]), n(ug["all_map"]), n(ug["plane_depth"]), W, Hh, cam.tanfovx, cam.tanfovy)
    got = n(grads[0][1][0])
    assert np.linalg.norm(got[:, :2] - rb["dL_dmeans2D"][:, :2]) <= 1e-3 * np.linalg.norm(rb["dL_dmeans2D"][:, :2])


def test_equal_depths_keep_emission_order(orc, H):
    """Many Gaussians at exactly the same depth: within a tile their order is the emission order (Gaussian index),
    whichever route builds the list."""
    import gs_scenes
    import gsrast_native as gn
    from diff_gaussian_rasterization import _C
    g, cams = gs_scenes.make_scene(0, P=20_000, n_views=1)
    cam = cams[0]
    W, Hh = cam.image_width, cam.image_height
    gx, gy = H.grid(W, Hh)
    o, gd = H.preprocess_fwd(g, cam)
    o["depths"] = (o["depths"] * 4).round() / 4  # few distinct values
    cl = torch.ones(gy, gx, dtype=torch.bool)
    n = lambda t: t.detach().cpu().numpy()
    want = orc.bin_and_sort(n(o["radii"]), n(o["means2D"]), n(o["depths"]), cl.numpy().reshape(-1), W, Hh)
    vm, cp = cam.world_view_transform.to(DEV), cam.camera_center.to(DEV)
    am = gs_scenes.build_all_map(gd["means3D"], gd["scales"], gd["rotations"], cam)
    for large, chunks in ROUTES:
        out = _C.render_gaussians(torch.zeros(3, device=DEV), Hh, W, o["means2D"], o["depths"], o["radii"],
                                  o["conic_opacity"], o["rgb"], cl.to(DEV), vm, cp, cam.tanfovx, cam.tanfovy, am,
                                  True, False, {"stats_collector": {}, "tile_sort_limits": (large, chunks)})
        R, binB = out[0], out[9]
        off = [C.c_size_t() for _ in range(5)]
        gn.check(gn.lib.gs_binning_state_layout(R, W, Hh, *[C.byref(x) for x in off]), "layout")
        base = (binB.data_ptr() + 255) // 256 * 256 - binB.data_ptr()
        point_list = binB[base + off[0].value: base + off[0].value + 4 * R].view(torch.int32)
        assert np.array_equal(H.np_u32(point_list), want["point_list"]), (large, chunks)


@pytest.mark.parametrize("P,expect", [(28_000, "mid"), (56_000, "long"), (110_000, "long2"),
                                      (110_000, "radix"), (230_000, "blocks"), (230_000, "blocks4k")])
def test_long_lists(orc, H, P, expect):
    """A small image under many large Gaussians: lists of several thousand records per tile.  Up to 4096 the
    smaller kernel of the per-tile radix sort takes them, up to 16384 the larger one, both inside the CU; beyond
    that (or beyond the block size the call asks for) the larger kernel sorts block by block through memory."""
    import gs_scenes
    import gsrast_native as gn
    from diff_gaussian_rasterization import _C
    g, cams = gs_scenes.make_scene(0, P=P, n_views=1)
    cam = cams[0]
    W, Hh = cam.image_width, cam.image_height
    gx, gy = H.grid(W, Hh)
    T = gx * gy
    g["scales"] = g["scales"] + 0.9  # larger splats: more tiles per Gaussian
    o, gd = H.preprocess_fwd(g, cam)
    cl = torch.ones(gy, gx, dtype=torch.bool)
    n = lambda t: t.detach().cpu().numpy()
    want = orc.bin_and_sort(n(o["radii"]), n(o["means2D"]), n(o["depths"]), cl.numpy().reshape(-1), W, Hh)
    counts = want["ranges"].reshape(-1, 2).astype(np.int64)
    longest = int((counts[:, 1] - counts[:, 0]).max())
    lo, hi = {"mid": (2048, 4096), "long": (4096, 8192), "long2": (8192, 16384), "radix": (8192, 16384),
              "blocks": (16384, 65536), "blocks4k": (16384, 65536)}[expect]
    assert lo < longest <= hi, longest
    limits = None
    if expect == "radix":
        limits = (0, 0)
    elif expect == "blocks4k":
        limits = (-1, 5000)
    vm, cp = cam.world_view_transform.to(DEV), cam.camera_center.to(DEV)
    am = gs_scenes.build_all_map(gd["means3D"], gd["scales"], gd["rotations"], cam)
    out = _C.render_gaussians(torch.zeros(3, device=DEV), Hh, W, o["means2D"], o["depths"], o["radii"],
                              o["conic_opacity"], o["rgb"], cl.to(DEV), vm, cp, cam.tanfovx, cam.tanfovy, am, True,
                              False, {"stats_collector": {}, "tile_sort_limits": limits})
    R, binB, imgB = out[0], out[9], out[10]
    assert R == want["point_list"].shape[0]
    off = [C.c_size_t() for _ in range(5)]
    gn.check(gn.lib.gs_binning_state_layout(R, W, Hh, *[C.byref(x) for x in off]), "layout")
    base = (binB.data_ptr() + 255) // 256 * 256 - binB.data_ptr()
    point_list = binB[base + off[0].value: base + off[0].value + 4 * R].view(torch.int32)
    keys = binB[base + off[1].value: base + off[1].value + 8 * R].view(torch.int64)
    ioff = [C.c_size_t() for _ in range(5)]
    gn.check(gn.lib.gs_image_state_layout(W, Hh, *[C.byref(x) for x in ioff]), "layout")
    ibase = (imgB.data_ptr() + 255) // 256 * 256 - imgB.data_ptr()
    ranges = imgB[ibase + ioff[3].value: ibase + ioff[3].value + 8 * T].view(torch.int32)
    assert np.array_equal(H.np_u32(ranges), want["ranges"].reshape(-1))
    assert np.array_equal(H.np_u64(keys), want["keys"])
    assert np.array_equal(H.np_u32(point_list), want["point_list"])


def test_grid_too_large_for_the_tile_histogram(orc, H):
    """3840x2160 is 32400 tiles, more than the counting kernels keep in LDS: the radix route is taken from the start."""
    import gs_scenes
    import gsrast_native as gn
    from diff_gaussian_rasterization import _C
    cam = gs_scenes.look_at_camera((0.0, 0.0, -30.0), (0, 0, 0), 3840, 2160, 60.0, up=(0.0, -1.0, 0.0))
    g, _ = gs_scenes.make_scene(0, P=20_000, n_views=1)
    W, Hh = cam.image_width, cam.image_height
    gx, gy = H.grid(W, Hh)
    T = gx * gy
    assert T > 30000
    o, gd = H.preprocess_fwd(g, cam)
    cl = torch.ones(gy, gx, dtype=torch.bool)
    n = lambda t: t.detach().cpu().numpy()
    want = orc.bin_and_sort(n(o["radii"]), n(o["means2D"]), n(o["depths"]), cl.numpy().reshape(-1), W, Hh)
    assert want["point_list"].shape[0] > 1000
    vm, cp = cam.world_view_transform.to(DEV), cam.camera_center.to(DEV)
    am = gs_scenes.build_all_map(gd["means3D"], gd["scales"], gd["rotations"], cam)
    out = _C.render_gaussians(torch.zeros(3, device=DEV), Hh, W, o["means2D"], o["depths"], o["radii"],
                              o["conic_opacity"], o["rgb"], cl.to(DEV), vm, cp, cam.tanfovx, cam.tanfovy, am, True,
                              False, {"stats_collector": {}})
    R, binB, imgB = out[0], out[9], out[10]
    assert R == want["point_list"].shape[0]
    off = [C.c_size_t() for _ in range(5)]
    gn.check(gn.lib.gs_binning_state_layout(R, W, Hh, *[C.byref(x) for x in off]), "layout")
    base = (binB.data_ptr() + 255) // 256 * 256 - binB.data_ptr()
    point_list = binB[base + off[0].value: base + off[0].value + 4 * R].view(torch.int32)
    ioff = [C.c_size_t() for _ in range(5)]
    gn.check(gn.lib.gs_image_state_layout(W, Hh, *[C.byref(x) for x in ioff]), "layout")
    ibase = (imgB.data_ptr() + 255) // 256 * 256 - imgB.data_ptr()
    ranges = imgB[ibase + ioff[3].value: ibase + ioff[3].value + 8 * T].view(torch.int32)
    assert np.array_equal(H.np_u32(ranges), want["ranges"].reshape(-1))
    assert np.array_equal(H.np_u32(point_list), want["point_list"])


@pytest.mark.parametrize("limits", [(-1, -1), (0, 0)])
def test_more_instances_than_positions_is_an_error(H, limits):
    """1.2 M splats that each cover all 3888 tiles are 4.7e9 instances: the 32-bit prefix sums wrap around to a
    plausible count (3.7e8).  The call must fail on the exact count instead of sizing its buffers by the wrapped
    one, whichever kernels did the counting."""
    import gsrast_native as gn
    from diff_gaussian_rasterization import _C
    P, W, Hh = 1_200_000, 1152, 864
    gx, gy = H.grid(W, Hh)
    assert P * gx * gy > 2 ** 32 and (P * gx * gy) % 2 ** 32 < 2 ** 31 - 2
    means2D = torch.full((P, 2), 500.0, device=DEV)
    depths = torch.ones(P, device=DEV)
    radii = torch.full((P,), 5000, dtype=torch.int32, device=DEV)
    co = torch.tensor([0.01, 0.0, 0.01, 0.5], device=DEV).repeat(P, 1)
    rgb = torch.zeros(P, 3, device=DEV)
    cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
    eye = torch.eye(4, device=DEV)
    with pytest.raises(RuntimeError, match="instances"):
        _C.render_gaussians(torch.zeros(3, device=DEV), Hh, W, means2D, depths, radii, co, rgb, cl, eye,
                            torch.zeros(3, device=DEV), 1.0, 0.75, torch.zeros(P, 5, device=DEV), False, False,
                            {"stats_collector": {}, "tile_sort_limits": limits})
    # a count just inside the limit is still served (here: none at all after the failed call)
    radii.zero_()
    out = _C.render_gaussians(torch.zeros(3, device=DEV), Hh, W, means2D, depths, radii, co, rgb, cl, eye,
                              torch.zeros(3, device=DEV), 1.0, 0.75, torch.zeros(P, 5, device=DEV), False, False,
                              {"stats_collector": {}, "tile_sort_limits": limits})
    assert out[0] == 0


@pytest.mark.parametrize("seed,W,Hh", [(0, 333, 217), (1, 1152, 864), (2, 64, 48), (3, 1920, 1080), (4, 17, 500)])
def test_random_rectangles_by_every_route(orc, H, seed, W, Hh):
    """Arbitrary splats handed straight to render_gaussians: radii from 0 to far beyond the image, centres inside,
    outside and non-finite, many equal depths, a random tile mask, image sizes that leave partial tiles.  Every
    route must build the oracle's lists."""
    import gsrast_native as gn
    from diff_gaussian_rasterization import _C
    gen = torch.Generator().manual_seed(seed)
    P = 6000
    gx, gy = H.grid(W, Hh)
    T = gx * gy
    means2D = torch.rand(P, 2, generator=gen) * torch.tensor([1.4 * W, 1.4 * Hh]) - torch.tensor([0.2 * W, 0.2 * Hh])
    kind = torch.randint(0, 10, (P,), generator=gen)
    radii = torch.randint(1, 12, (P,), generator=gen, dtype=torch.int32)
    radii[kind == 0] = 0
    radii[kind == 1] = torch.randint(40, 200, (int((kind == 1).sum()),), generator=gen, dtype=torch.int32)
    radii[kind == 2] = 100000  # covers every tile
    radii[kind == 3] = 2 ** 31 - 1
    means2D[kind == 4, 0] = float("nan")
    means2D[kind == 5, 1] = float("inf")
    means2D[kind == 6] = -1e30
    depths = (torch.rand(P, generator=gen) * 8).round() / 2 + 0.5  # 17 distinct values
    cl = torch.rand(gy, gx, generator=gen) < 0.7
    n = lambda t: t.detach().cpu().numpy()
    want = orc.bin_and_sort(n(radii), n(means2D), n(depths), cl.numpy().reshape(-1), W, Hh)
    R_want = int(want["point_list"].shape[0])
    assert R_want > T  # the splats that cover everything alone give that
    co = torch.tensor([0.02, 0.0, 0.02, 0.3]).repeat(P, 1).to(DEV)
    rgb = torch.rand(P, 3, generator=gen).to(DEV)
    eye = torch.eye(4, device=DEV)
    for large, chunks in ROUTES:
        out = _C.render_gaussians(torch.zeros(3, device=DEV), Hh, W, means2D.to(DEV), depths.to(DEV), radii.to(DEV),
                                  co, rgb, cl.to(DEV), eye, torch.zeros(3, device=DEV), 1.0, 1.0,
                                  torch.zeros(P, 5, device=DEV), False, False,
                                  {"stats_collector": {}, "tile_sort_limits": (large, chunks)})
        R, binB, imgB = out[0], out[9], out[10]
        assert R == R_want, (large, chunks)
        off = [C.c_size_t() for _ in range(5)]
        gn.check(gn.lib.gs_binning_state_layout(R, W, Hh, *[C.byref(x) for x in off]), "layout")
        base = (binB.data_ptr() + 255) // 256 * 256 - binB.data_ptr()
        point_list = binB[base + off[0].value: base + off[0].value + 4 * R].view(torch.int32)
        keys = binB[base + off[1].value: base + off[1].value + 8 * R].view(torch.int64)
        ioff = [C.c_size_t() for _ in range(5)]
        gn.check(gn.lib.gs_image_state_layout(W, Hh, *[C.byref(x) for x in ioff]), "layout")
        ibase = (imgB.data_ptr() + 255) // 256 * 256 - imgB.data_ptr()
        ranges = imgB[ibase + ioff[3].value: ibase + ioff[3].value + 8 * T].view(torch.int32)
        assert np.array_equal(H.np_u32(ranges), want["ranges"].reshape(-1)), (large, chunks)
        assert np.array_equal(H.np_u64(keys), want["keys"]), (large, chunks)
        assert np.array_equal(H.np_u32(point_list), want["point_list"]), (large, chunks)


@pytest.mark.parametrize("P", [1500, 3500, 9000, 20000])
def test_depths_that_agree_in_their_leading_bits(orc, H, P):
    """The per-tile sorts order their lists on the leading bits of the depth (relative to the list's smallest) and
    leave the rest to their last step.  Here every splat covers every tile and the depths form two clusters, at 1
    and at 64, whose members differ in their last 9 bits only (some not at all): all of a cluster shares the
    leading bits at every list length (registers, both radix kernels, a split list), so the whole order inside a
    cluster is made by that last step, by all depth bits and then the emission index."""
    import gsrast_native as gn
    from diff_gaussian_rasterization import _C
    gen = torch.Generator().manual_seed(P)
    W, Hh = 64, 48
    gx, gy = H.grid(W, Hh)
    T = gx * gy
    means2D = torch.rand(P, 2, generator=gen) * torch.tensor([float(W), float(Hh)])
    radii = torch.full((P,), 1000, dtype=torch.int32)
    base = torch.where(torch.rand(P, generator=gen) < 0.5, torch.tensor(1.0), torch.tensor(64.0))
    ulps = torch.randint(0, 300, (P,), generator=gen, dtype=torch.int32)
    depths = (base.view(torch.int32) + ulps).view(torch.float32)
    cl = torch.ones(gy, gx, dtype=torch.bool)
    n = lambda t: t.detach().cpu().numpy()
    want = orc.bin_and_sort(n(radii), n(means2D), n(depths), cl.numpy().reshape(-1), W, Hh)
    assert int(want["point_list"].shape[0]) == P * T
    co = torch.tensor([0.02, 0.0, 0.02, 0.3]).repeat(P, 1).to(DEV)
    eye = torch.eye(4, device=DEV)
    out = _C.render_gaussians(torch.zeros(3, device=DEV), Hh, W, means2D.to(DEV), depths.to(DEV), radii.to(DEV), co,
                              torch.zeros(P, 3, device=DEV), cl.to(DEV), eye, torch.zeros(3, device=DEV), 1.0, 1.0,
                              torch.zeros(P, 5, device=DEV), False, False, {"stats_collector": {}})
    R, binB, imgB = out[0], out[9], out[10]
    assert R == P * T
    off = [C.c_size_t() for _ in range(5)]
    gn.check(gn.lib.gs_binning_state_layout(R, W, Hh, *[C.byref(x) for x in off]), "layout")
    b0 = (binB.data_ptr() + 255) // 256 * 256 - binB.data_ptr()
    point_list = binB[b0 + off[0].value: b0 + off[0].value + 4 * R].view(torch.int32)
    keys = binB[b0 + off[1].value: b0 + off[1].value + 8 * R].view(torch.int64)
    assert np.array_equal(H.np_u64(keys), want["keys"])
    assert np.array_equal(H.np_u32(point_list), want["point_list"])
