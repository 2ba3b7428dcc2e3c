"""BASELINE configurations 2, 3 and 4 on the GPU.

Two kinds of test per configuration:
  * its distribution (scene statistics, cameras, image size) at a reduced Gaussian count, EVERY camera of the batch
    (the reference loops over the cameras of a batch, gaussian_renderer/__init__.py:966-1023), the whole step
    (preprocess, per-tile lists, blend forward and backward, preprocess backward) against the CPU oracle;
  * its full size (4 M x 4 views, 10 M x 8 views at 1920x1080, 20 M x 4 views with simple-knn, densification
    statistics and the optimizer step) through properties that need no CPU run of that size.
"""
import ctypes as C
import time

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
IMG_BYTES = True  # forward images are compared bit for bit


@pytest.fixture(scope="module")
def H():
    import gpu_harness
    return gpu_harness


def _settings(cam, bg):
    from diff_gaussian_rasterization import GaussianRasterizationSettings
    return GaussianRasterizationSettings(
        image_height=cam.image_height, image_width=cam.image_width, tanfovx=cam.tanfovx, tanfovy=cam.tanfovy,
        bg=torch.tensor(bg, dtype=torch.float32, device=DEV), scale_modifier=1.0,
        viewmatrix=cam.world_view_transform.to(DEV), projmatrix=cam.full_proj_transform.to(DEV), sh_degree=3,
        campos=cam.camera_center.to(DEV), prefiltered=False, render_geo=True, debug=False)


def _tmp_mask(out_all_map, cam):
    """Pixels whose plane-depth denominator (blended normal . ray) is at least 1e-3 in size: elsewhere the
    plane-depth gradient is astronomically large and carries no information about parity."""
    W, Hh = cam.image_width, cam.image_height
    fx, fy = W / (2.0 * cam.tanfovx), Hh / (2.0 * cam.tanfovy)
    rayx = (np.arange(W, dtype=np.float64)[None, :] - W * 0.5) / fx
    rayy = (np.arange(Hh, dtype=np.float64)[:, None] - Hh * 0.5) / fy
    om = out_all_map.astype(np.float64)
    return np.abs(om[0] * rayx + om[1] * rayy + om[2]) >= 1e-3


@pytest.mark.timeout(600)
@pytest.mark.parametrize("cfg,P,views", [(2, 400_000, 4), (3, 150_000, 8), (4, 400_000, 4)])
def test_every_view_of_the_batch_matches_the_oracle(orc, H, cfg, P, views):
    import gs_scenes
    from diff_gaussian_rasterization import GaussianRasterizer
    g, cams = gs_scenes.make_scene(cfg, P=P)
    assert len(cams) == views
    n = lambda t: t.detach().cpu().numpy()
    gnp = {k: n(g[k]) for k in ("means3D", "scales", "rotations", "opacities", "shs")}
    bg = (0.1, 0.3, 0.2)
    bgn = np.array(bg, np.float32)
    total_R = 0
    for v, cam in enumerate(cams):
        tag = f"config {cfg} view {v}"
        W, Hh = cam.image_width, cam.image_height
        gx, gy = H.grid(W, Hh)
        rast = GaussianRasterizer(_settings(cam, bg))
        leaf = {k: g[k].to(DEV).requires_grad_(True) for k in gnp}
        args = {"stats_collector": {}, "max_weight_depth": cfg == 2}
        means2D, rgb, co, radii, depths = rast.preprocess_gaussians(leaf["means3D"], leaf["scales"], leaf["rotations"],
                                                                    leaf["shs"], leaf["opacities"], args)
        for t in (means2D, co, rgb):
            t.retain_grad()
        am = gs_scenes.build_all_map(g["means3D"], g["scales"], g["rotations"], cam).to(DEV).requires_grad_(True)
        cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
        m2abs = torch.zeros(P, 3, device=DEV, requires_grad=True)
        color, n_render, n_consider, n_contrib, obs, oam, opd = rast.render_gaussians(
            means2D, m2abs, co, rgb, am, depths, radii, cl, cl, args)

        Vn, PMn, cpn = n(cam.world_view_transform), n(cam.full_proj_transform), n(cam.camera_center)
        pre = orc.preprocess_fwd(gnp["means3D"], gnp["scales"], gnp["rotations"], gnp["opacities"], gnp["shs"], Vn,
                                 PMn, cpn, W, Hh, cam.tanfovx, cam.tanfovy)
        assert np.array_equal(n(radii), pre["radii"]), tag
        for k, t in (("means2D", means2D), ("conic_opacity", co), ("rgb", rgb), ("depths", depths)):
            assert np.array_equal(n(t), pre[k]), (tag, k)
        cln = np.ones(gx * gy, bool)
        b = orc.bin_and_sort(pre["radii"], pre["means2D"], pre["depths"], cln, W, Hh)
        total_R += b["num_rendered"]
        f = orc.render_fwd(b["ranges"], b["point_list"], pre["means2D"], pre["rgb"], n(am), pre["conic_opacity"], cln,
                           bgn, W, Hh, cam.tanfovx, cam.tanfovy)
        for got, want in ((n_render, "n_render"), (n_consider, "n_consider"), (n_contrib, "n_contrib_tile"),
                          (obs, "out_observe")):
            assert np.array_equal(n(got), f[want]), (tag, want)
        assert np.array_equal(n(color), f["color"]), tag
        assert np.array_equal(n(oam), f["out_all_map"]), tag
        a, r = n(opd), f["out_plane_depth"]
        assert np.array_equal(np.isnan(a), np.isnan(r)) and np.array_equal(a[~np.isnan(r)], r[~np.isnan(r)]), tag
        if cfg == 2:
            want = orc.max_weight_depth(b["ranges"], b["point_list"], pre["means2D"], pre["conic_opacity"],
                                        pre["depths"], cln, W, Hh)
            assert np.array_equal(n(args["stats_collector"]["max_weight_depth"]), want), tag

        ug = gs_scenes.upstream_grads(cam, seed=v)
        gdep = ug["plane_depth"] * torch.from_numpy(_tmp_mask(f["out_all_map"], cam)[None].astype(np.float32))
        torch.autograd.backward([color, oam, opd], [ug["color"].to(DEV), ug["all_map"].to(DEV), gdep.to(DEV)])
        rb = orc.render_bwd(b["ranges"], b["point_list"], pre["means2D"], pre["conic_opacity"], pre["rgb"], n(am),
                            f["out_all_map"], f["final_T"], f["n_contrib"], cln, bgn, n(ug["color"]),
                            n(ug["all_map"]), n(gdep), W, Hh, cam.tanfovx, cam.tanfovy)
        pb = orc.preprocess_bwd(gnp["means3D"], pre["radii"], gnp["shs"], pre["clamped"], gnp["scales"],
                                gnp["rotations"], pre["cov3D"], Vn, PMn, cpn, W, Hh, cam.tanfovx, cam.tanfovy,
                                rb["dL_dmeans2D"], rb["dL_dconic_opacity"], rb["dL_dcolors"])
        def close(k, got, want, rel, per_element):
            a = n(got).reshape(want.shape)
            assert np.isfinite(a).all(), (tag, k)
            assert H.rel_l2(a, want) <= rel, (tag, k, H.rel_l2(a, want))
            if per_element:
                # each element within `rel` of its own size plus 1e-5 of the tensor's largest: a wrong gradient of
                # a Gaussian with a small one cannot hide behind the large ones
                worst = np.abs(a - want) - (rel * np.abs(want) + 1e-5 * np.abs(want).max())
                assert worst.max() <= 0.0, (tag, k, float(worst.max()))

        # the blend's own gradients against the oracle's, element by element
        close("means2D", means2D.grad, rb["dL_dmeans2D"][:, :2], 1e-3, True)
        close("means2D_abs", m2abs.grad, rb["dL_dmeans2D_abs"], 1e-3, True)
        close("conic_opacity", co.grad, rb["dL_dconic_opacity"], 1e-3, True)
        close("rgb", rgb.grad, rb["dL_dcolors"], 1e-3, True)
        close("all_map", am.grad, rb["dL_dall_map"], 1e-3, True)
        # the per-Gaussian backward on the very gradients the GPU blend produced: the same operations in the same
        # order as the oracle's, element by element
        pg = orc.preprocess_bwd(gnp["means3D"], pre["radii"], gnp["shs"], pre["clamped"], gnp["scales"],
                                gnp["rotations"], pre["cov3D"], Vn, PMn, cpn, W, Hh, cam.tanfovx, cam.tanfovy,
                                n(means2D.grad), n(co.grad), n(rgb.grad))
        leaves = (("means3D", "dL_dmeans3D"), ("scales", "dL_dscales"), ("rotations", "dL_drotations"),
                  ("opacities", "dL_dopacity"), ("shs", "dL_dsh"))
        for k, r in leaves:
            close(k, leaf[k].grad, pg[r], 1e-5, True)
        # and the whole chain against the oracle's whole chain (rows with cancelling terms amplify the blend's
        # summation-order differences, so this one is a norm)
        for k, r in leaves:
            close(k + " (chain)", leaf[k].grad, pb[r], 1e-3, False)
    assert total_R > views * 10_000  # the cameras do look at the scene


def _buffer_views(gn, geomB, binB, imgB, P, R, W, Hh, T):
    off = [C.c_size_t() for _ in range(5)]
    gn.check(gn.lib.gs_binning_state_layout(R, W, Hh, *[C.byref(o) for o in off]), "layout")
    base = (binB.data_ptr() + 255) // 256 * 256 - binB.data_ptr()
    point_list = binB[base + off[0].value: base + off[0].value + 4 * R].view(torch.int32)
    keys = binB[base + off[1].value: base + off[1].value + 8 * R].view(torch.int64)
    goff = [C.c_size_t() for _ in range(3)]
    gn.check(gn.lib.gs_geometry_state_layout(P, *[C.byref(o) for o in goff]), "layout")
    gbase = (geomB.data_ptr() + 255) // 256 * 256 - geomB.data_ptr()
    tiles_touched = geomB[gbase + goff[0].value: gbase + goff[0].value + 4 * P].view(torch.int32)
    ioff = [C.c_size_t() for _ in range(5)]
    gn.check(gn.lib.gs_image_state_layout(W, Hh, *[C.byref(o) for o in ioff]), "layout")
    ibase = (imgB.data_ptr() + 255) // 256 * 256 - imgB.data_ptr()
    final_T = imgB[ibase + ioff[0].value: ibase + ioff[0].value + 4 * W * Hh].view(torch.float32)
    return point_list, keys, tiles_touched, final_T


def _full_size_view(H, d, cam, view, render_geo=True, args=None, scale_modifier=1.0):
    """One view of a full-size configuration, forward and backward, checked through properties: list order and
    counts, image ranges, repeatability bit for bit forward, linearity and exact zeros backward.  Returns what the
    caller's later stages use."""
    import gs_scenes
    import gsrast_native as gn
    from diff_gaussian_rasterization import _C
    tag = f"view {view}"
    W, Hh = cam.image_width, cam.image_height
    P = d["means3D"].shape[0]
    vm, pm, cp = cam.world_view_transform.to(DEV), cam.full_proj_transform.to(DEV), cam.camera_center.to(DEV)
    args = args if args is not None else {"stats_collector": {}}
    gx, gy = (W + 15) // 16, (Hh + 15) // 16
    T = gx * gy
    cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
    _, means2D, depths, radii, cov3D, co, rgb, clamped = _C.preprocess_gaussians(
        d["means3D"], d["scales"], d["rotations"], d["shs"], d["opacities"], scale_modifier, vm, pm, cam.tanfovx,
        cam.tanfovy, Hh, W, 3, cp, False, False, args)
    am = _C.build_all_map(d["means3D"], d["scales"], d["rotations"], vm, cp)
    bg = torch.zeros(3, device=DEV)

    def forward():
        return _C.render_gaussians(bg, Hh, W, means2D, depths, radii, co, rgb, cl, vm, cp, cam.tanfovx, cam.tanfovy,
                                   am, render_geo, False, args)

    out = forward()
    R, color, n_render, n_consider, n_contrib, out_observe, oam, opd, geomB, binB, imgB = out
    assert R > 100_000 and int(n_render.sum()) == R, tag
    point_list, keys, tiles_touched, final_T = _buffer_views(gn, geomB, binB, imgB, P, R, W, Hh, T)
    end_bit = 32 + gn.lib.gs_higher_msb(T)
    masked = keys & ((1 << end_bit) - 1)
    assert bool((masked[1:] >= masked[:-1]).all()), tag
    tile_of = masked >> 32
    assert int(tile_of.max()) < T, tag
    assert bool((torch.bincount(tile_of, minlength=T) == n_render.to(torch.int64)).all()), tag
    assert bool((torch.bincount(point_list.to(torch.int64), minlength=P) == tiles_touched.to(torch.int64)).all()), tag
    assert bool((tiles_touched[radii == 0] == 0).all()), tag
    # the key's low word is the depth of the Gaussian at that position, and equal keys keep emission (= Gaussian) order
    assert bool(((masked & 0xFFFFFFFF).to(torch.int32) == depths[point_list.to(torch.int64)].view(torch.int32)).all()), tag
    same = masked[1:] == masked[:-1]
    assert bool((point_list[1:][same] > point_list[:-1][same]).all()), tag
    del masked, tile_of, same
    assert bool(torch.isfinite(color).all()) and bool(torch.isfinite(oam).all()), tag
    assert float(final_T.min()) >= 0.0 and float(final_T.max()) <= 1.0, tag
    assert bool((color >= 0).all()), tag
    assert int(out_observe.sum()) <= int(n_contrib.sum()) <= int(n_consider.sum()), tag
    if render_geo:
        # alpha channel of the blended geometry map: 1 - final transmittance (the channel is 1 for every Gaussian)
        assert float((oam[3] - (1.0 - final_T.view(Hh, W))).abs().max()) <= 1e-4, tag
    out2 = forward()
    for a, b in zip(out[:8], out2[:8]):
        assert torch.equal(a, b) if torch.is_tensor(a) else a == b, tag
    del out2

    ug = gs_scenes.upstream_grads(cam, seed=view)
    gc, ga, gd = ug["color"].to(DEV), ug["all_map"].to(DEV), ug["plane_depth"].to(DEV)
    if render_geo:
        # keep the plane-depth gradient where its denominator (blended normal . ray) is not tiny
        fx, fy = W / (2.0 * cam.tanfovx), Hh / (2.0 * cam.tanfovy)
        rx = (torch.arange(W, device=DEV, dtype=torch.float64)[None, :] - W * 0.5) / fx
        ry = (torch.arange(Hh, device=DEV, dtype=torch.float64)[:, None] - Hh * 0.5) / fy
        tmp = oam[0].double() * rx + oam[1].double() * ry + oam[2].double()
        gd = gd * (tmp.abs() >= 1e-3)[None].float()

    def backward(scale):
        return _C.render_gaussians_backward(bg, cam.tanfovx, cam.tanfovy, oam, am, R, geomB, binB, imgB, cl,
                                            gc * scale, ga * scale, gd * scale, means2D, co, rgb, render_geo, False,
                                            args)

    b1, b1r, b2 = backward(1.0), backward(1.0), backward(2.0)
    for x, y, z in zip(b1, b1r, b2):
        assert bool(torch.isfinite(x).all()), tag
        assert torch.equal(x, y), tag  # every sum is taken in a fixed order: the same bits from run to run
        nx = float(x.double().norm())
        assert float((2.0 * x.double() - z.double()).norm()) <= 1e-5 * 2 * nx, tag
    dead = radii == 0
    for t in b1:
        assert float(t[dead].abs().max()) == 0.0, tag
    assert bool((b1[1][:, :2] * (1 + 1e-3) + 1e-6 >= b1[0].abs()).all()) and float(b1[1][:, 2].abs().max()) == 0.0, tag
    pb = _C.preprocess_gaussians_backward(radii, cov3D, clamped, d["means3D"], d["scales"], d["rotations"], d["shs"],
                                          scale_modifier, vm, pm, cam.tanfovx, cam.tanfovy, Hh, W, 3, cp, b1[0], b1[2],
                                          b1[3], R, False, args)
    for t in pb:
        assert bool(torch.isfinite(t).all()), tag
        assert float(t[dead].abs().max()) == 0.0, tag
    return dict(R=R, longest=int(n_render.max()), radii=radii, means2D_grad=b1[0], grads=pb, color=color)


def _load(cfg):
    import gs_scenes
    g, cams = gs_scenes.make_scene(cfg)
    d = {k: v.to(DEV) for k, v in g.items() if torch.is_tensor(v)}
    del g
    return d, cams


@pytest.mark.timeout(900)
def test_config2_full_size_all_views(H):
    """4 M Gaussians (70 % within a few metres of the ground), four cameras on the 300 m circle, 1152x864, geometry
    maps and the per-pixel depth of the heaviest Gaussian."""
    d, cams = _load(2)
    assert d["means3D"].shape[0] == 4_000_000 and len(cams) == 4
    for v, cam in enumerate(cams):
        args = {"stats_collector": {}, "max_weight_depth": True}
        r = _full_size_view(H, d, cam, v, args=args)
        mwd = args["stats_collector"]["max_weight_depth"]
        assert mwd.shape == (1, cam.image_height, cam.image_width) and bool(torch.isfinite(mwd).all())
        # a depth of some visible Gaussian wherever anything was blended, 0 elsewhere
        assert float(mwd.min()) >= 0.0 and float(mwd.max()) > 100.0
        assert r["R"] > 1_000_000


@pytest.mark.timeout(900)
def test_config3_full_size_all_views_forward_and_backward_with_geometry(H):
    """10 M Gaussians, eight street-level cameras (2 m above the ground), 1920x1080: lists of more than 8192
    records, Gaussians that cover thousands of tiles; forward and backward with the geometry maps on."""
    d, cams = _load(3)
    assert d["means3D"].shape[0] == 10_000_000 and len(cams) == 8
    longest = 0
    for v, cam in enumerate(cams):
        assert (cam.image_width, cam.image_height) == (1920, 1080)
        r = _full_size_view(H, d, cam, v)
        longest = max(longest, r["longest"])
    assert longest > 8192  # the regime of the per-tile radix sort's larger kernel


@pytest.mark.timeout(900)
def test_config3_hundred_million_instances(H):
    """The regime BASELINE config 3 names (lists of more than 5000 Gaussians per tile, more than 100 M keys), which
    its own generator stays a factor 12 below: the street-level view with the most instances, its Gaussians enlarged
    by the rasterizer's scale modifier until the view has at least 10^8 instances; forward and backward with the
    geometry maps through the property checks of every full-size view.  Positions, layouts and record indices
    are 32-bit up to 2^31-2 instances; this view exercises them at a twentieth of that."""
    import gsrast_native as gn
    from diff_gaussian_rasterization import _C
    d, cams = _load(3)
    cam = cams[6]
    W, Hh = cam.image_width, cam.image_height
    P = d["means3D"].shape[0]
    vm, pm, cp = cam.world_view_transform.to(DEV), cam.full_proj_transform.to(DEV), cam.camera_center.to(DEV)
    gx, gy = (W + 15) // 16, (Hh + 15) // 16
    cl = torch.ones(gy * gx, dtype=torch.bool, device=DEV)
    tt = torch.empty(P, dtype=torch.int32, device=DEV)
    mod, R = 2.0, 0
    while True:
        _, means2D, depths, radii, _, _, _, _ = _C.preprocess_gaussians(
            d["means3D"], d["scales"], d["rotations"], d["shs"], d["opacities"], mod, vm, pm, cam.tanfovx, cam.tanfovy,
            Hh, W, 3, cp, False, False, {})
        gn.check(gn.lib.gs_tile_count(P, W, Hh, H.ptr(radii), H.ptr(means2D), H.ptr(cl), H.ptr(tt), H.stream()),
                 "gs_tile_count")
        R = int(tt.to(torch.int64).sum())
        if R >= 100_000_000:
            break
        assert mod < 40.0, (mod, R)
        mod *= 1.25 if R > 50_000_000 else 1.5
    del means2D, depths, radii, tt
    assert R < 400_000_000, (mod, R)  # (a few tens of GB of buffers at most)
    print(f"scale modifier {mod:.3f}: {R} instances", flush=True)
    gn.stage_timing(True)
    r = _full_size_view(H, d, cam, 6, scale_modifier=mod)
    torch.cuda.synchronize()
    gn.stage_timing(False)
    st = gn.stage_timing_collect()
    assert r["R"] == R and r["longest"] > 16384
    print("stages (ms per launch, launches): " +
          ", ".join(f"{k} {tot / max(cnt, 1):.3f} x{cnt}" for k, (tot, cnt) in st.items()), flush=True)
    print(f"longest list {r['longest']}", flush=True)


@pytest.mark.timeout(1100)
def test_config4_full_size_iteration(H):
    """20 M Gaussians: simple-knn over all means (initialisation), four views forward and backward, the
    densification statistics and the running maximum of the radii per view, and one fused Adam step over all five
    parameter tensors with the gradients summed over the views."""
    import gs_densify
    from gs_optim import FusedAdam
    from simple_knn._C import distCUDA2
    d, cams = _load(4)
    P = d["means3D"].shape[0]
    assert P == 20_000_000 and len(cams) == 4

    # --- distCUDA2 over all 20 M means, 512 of them against an exhaustive search
    pts = d["means3D"]
    got = distCUDA2(pts)
    assert got.shape == (P,) and bool(torch.isfinite(got).all()) and float(got.min()) > 0.0
    gq = torch.Generator(device=DEV).manual_seed(4)
    q = torch.randint(0, P, (512,), generator=gq, device=DEV)
    best = torch.full((512, 3), float("inf"), device=DEV)
    for s in range(0, P, 500_000):
        blk = pts[s:s + 500_000]
        df = blk[None, :, :] - pts[q][:, None, :]
        d2 = (df[..., 0] * df[..., 0] + df[..., 1] * df[..., 1]) + df[..., 2] * df[..., 2]
        own = q[:, None] == (torch.arange(blk.shape[0], device=DEV)[None, :] + s)
        d2 = torch.where(own, torch.full_like(d2, float("inf")), d2)
        best = torch.cat([best, d2], dim=1).topk(3, dim=1, largest=False).values
        del df, d2, own
    want = ((best[:, 0] + best[:, 1]) + best[:, 2]) / 3.0
    assert float(((got[q] - want).abs() / want).max()) <= 1e-6
    del got, best

    # --- four views; per view the statistics the training loop keeps (train_internal.py:376-392).  The anchors
    # are the Gaussians themselves here (one offset each, every anchor visible, every candidate selected).
    acc = [torch.zeros(P, 1, device=DEV) for _ in range(4)]
    max_radii = torch.zeros(P, device=DEV)
    total = {k: torch.zeros_like(d[k]) for k in ("means3D", "scales", "rotations", "shs", "opacities")}
    seen = torch.zeros(P, dtype=torch.int32, device=DEV)
    norm_sum = torch.zeros(P, device=DEV)
    ones = torch.ones(P, dtype=torch.bool, device=DEV)
    for v, cam in enumerate(cams):
        r = _full_size_view(H, d, cam, v)
        flt = r["radii"] > 0
        g2 = torch.cat([r["means2D_grad"], torch.zeros(P, 1, device=DEV)], dim=1).contiguous()
        gs_densify.training_statis(acc[0], acc[1], acc[2], acc[3], 1, g2, d["opacities"], flt, ones, ones)
        gs_densify.update_max_radii(max_radii, r["radii"], flt)
        seen += flt.int()
        norm_sum += torch.where(flt, r["means2D_grad"].norm(dim=1), torch.zeros(P, device=DEV))
        for k, t in zip(("means3D", "scales", "rotations", "shs", "opacities"), r["grads"]):
            total[k] += t.reshape(total[k].shape)
        assert float(max_radii.max()) >= float(r["radii"].max())
        del r, g2
    assert torch.equal(acc[1].view(-1), torch.full((P,), 4.0, device=DEV))  # every anchor was visible four times
    assert torch.equal(acc[3].view(-1), seen.float())
    assert float((acc[2].view(-1) - norm_sum).abs().max()) <= 1e-5 * max(1.0, float(norm_sum.max()))
    assert float((acc[0].view(-1) - 4.0 * d["opacities"].view(-1).clamp(min=0)).abs().max()) <= 1e-5
    assert bool((max_radii[seen == 0] == 0).all()) and bool((max_radii[seen > 0] > 0).all())

    # --- one optimizer step over all five tensors (scene/gaussian_model.py:561-574 learning rates), gradients
    # averaged over the four views inside the update; a slice against torch.optim.Adam
    names = ("means3D", "scales", "rotations", "shs", "opacities")
    lrs = dict(means3D=1.6e-4, scales=5e-3, rotations=1e-3, shs=2.5e-3, opacities=5e-2)
    params = {k: d[k].clone().requires_grad_(True) for k in names}
    sl = slice(7_000_000, 7_050_000)
    theirs = {k: d[k][sl].clone().requires_grad_(True) for k in names}
    for k in names:
        params[k].grad = total[k]
        theirs[k].grad = total[k][sl] * 0.25
    mine = FusedAdam([{"params": [params[k]], "lr": lrs[k], "name": k} for k in names], lr=0.0, eps=1e-15,
                     grad_scale=0.25)
    ref = torch.optim.Adam([{"params": [theirs[k]], "lr": lrs[k], "name": k} for k in names], lr=0.0, eps=1e-15)
    mine.step()
    ref.step()
    moved = 0
    for k in names:
        a = (params[k].detach()[sl] - d[k][sl]).double()
        b = (theirs[k].detach() - d[k][sl]).double()
        assert float((a - b).norm()) <= 1e-5 * max(float(b.norm()), 1e-30), k
        assert bool(torch.isfinite(params[k]).all()), k
        untouched = total[k] == 0
        # eps = 1e-15: a parameter whose gradient is exactly zero does not move on the first step
        assert torch.equal(params[k].detach()[untouched], d[k][untouched]), k
        moved += int((params[k].detach() != d[k]).sum())
    assert moved > 1_000_000
