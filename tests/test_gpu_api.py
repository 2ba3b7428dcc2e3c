"""The Python operator API (GaussianRasterizationSettings / GaussianRasterizer /
distCUDA2) end to end on the GPU, with the call sequence CityGS-X uses
(visible_filter -> preprocess -> all_map in torch -> render -> backward), against
the CPU oracle running the same sequence."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _settings(cam, render_geo=True, sh_degree=3, bg=(0.0, 0.0, 0.0)):
    from diff_gaussian_rasterization import GaussianRasterizationSettings
    return GaussianRasterizationSettings(
        image_height=cam.image_height, image_width=cam.image_width, tanfovx=cam.tanfovx, tanfovy=cam.tanfovy,
        bg=torch.tensor(bg, dtype=torch.float32, device=DEV), scale_modifier=1.0,
        viewmatrix=cam.world_view_transform.to(DEV), projmatrix=cam.full_proj_transform.to(DEV), sh_degree=sh_degree,
        campos=cam.camera_center.to(DEV), prefiltered=False, render_geo=render_geo, debug=False)


def _cuda_args():
    return {"mode": "train", "global_rank": "0", "world_size": "1", "iteration": "1", "log_interval": "10",
            "log_folder": "/tmp", "zhx_debug": "False", "zhx_time": "False", "avoid_pixel_all2all": False,
            "stats_collector": {}}


def _rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


def test_block_xy_and_module_surface():
    import diff_gaussian_rasterization as dgr
    assert dgr._C.get_block_XY() == (16, 16, 256)
    with pytest.raises(RuntimeError, match="deprecated"):
        dgr._C.get_distribution_strategy()
    with pytest.raises(NotImplementedError):
        dgr._C.get_local2j_ids_bool()


@pytest.mark.parametrize("cfg,P,sh_mode", [(0, 50_000, True), (1, 150_000, True), (1, 150_000, False)])
def test_full_pipeline_matches_oracle(orc, cfg, P, sh_mode):
    import gs_scenes
    from diff_gaussian_rasterization import GaussianRasterizer
    g, cams = gs_scenes.make_scene(cfg, P=P, n_views=1)
    cam = cams[0]
    W, H = cam.image_width, cam.image_height
    rs = _settings(cam)
    rast = GaussianRasterizer(rs)
    leaf = {k: g[k].to(DEV).requires_grad_(True) for k in ("means3D", "scales", "rotations", "opacities", "shs")}
    mlp_rgb = torch.rand(P, 3, generator=torch.Generator().manual_seed(3)).to(DEV).requires_grad_(True)
    cuda_args = _cuda_args()

    vis = rast.visible_filter(leaf["means3D"].detach(), leaf["scales"].detach(), leaf["rotations"].detach())
    shs_arg = leaf["shs"] if sh_mode else mlp_rgb
    means2D, rgb, conic_opacity, radii, depths = rast.preprocess_gaussians(
        leaf["means3D"], leaf["scales"], leaf["rotations"], shs_arg, leaf["opacities"], cuda_args)
    assert means2D.shape == (P, 2) and rgb.shape == (P, 3) and conic_opacity.shape == (P, 4)
    assert radii.dtype == torch.int32 and radii.shape == (P,) and depths.shape == (P,)
    assert not radii.requires_grad and not depths.requires_grad
    assert torch.equal(vis, radii)
    means2D.retain_grad()
    all_map = gs_scenes.build_all_map(leaf["means3D"], leaf["scales"], leaf["rotations"], cam)
    gx, gy = (W + 15) // 16, (H + 15) // 16
    cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
    means2D_abs = torch.zeros_like(leaf["means3D"], requires_grad=True) + 0
    means2D_abs.retain_grad()
    colour_in = rgb if sh_mode else mlp_rgb
    color, n_render, n_consider, n_contrib, out_observe, out_all_map, out_plane_depth = rast.render_gaussians(
        means2D, means2D_abs, conic_opacity, colour_in, all_map, depths, radii, cl, cl, cuda_args)
    assert color.shape == (3, H, W) and out_all_map.shape == (5, H, W) and out_plane_depth.shape == (1, H, W)
    assert n_render.shape == (gx * gy,) and n_render.dtype == torch.int32 and out_observe.shape == (P,)
    assert "forward_render_time" in cuda_args["stats_collector"]
    ug = gs_scenes.upstream_grads(cam)
    loss = (color * ug["color"].to(DEV)).sum() + (out_all_map * ug["all_map"].to(DEV)).sum() + \
        (out_plane_depth * ug["plane_depth"].to(DEV)).sum()
    loss.backward()
    assert "backward_render_time" in cuda_args["stats_collector"]

    # ---- oracle, same sequence
    n = lambda t: t.detach().cpu().numpy()
    pre = orc.preprocess_fwd(n(g["means3D"]), n(g["scales"]), n(g["rotations"]), n(g["opacities"]),
                             n(g["shs"]) if sh_mode else None, n(cam.world_view_transform), n(cam.full_proj_transform),
                             n(cam.camera_center), W, H, cam.tanfovx, cam.tanfovy)
    assert np.array_equal(n(radii), pre["radii"])
    cl_np = np.ones(gx * gy, bool)
    b = orc.bin_and_sort(pre["radii"], pre["means2D"], pre["depths"], cl_np, W, H)
    am = n(all_map)
    col_np = pre["rgb"] if sh_mode else n(mlp_rgb)
    f = orc.render_fwd(b["ranges"], b["point_list"], pre["means2D"], col_np, am, pre["conic_opacity"], cl_np,
                       np.zeros(3, np.float32), W, H, cam.tanfovx, cam.tanfovy)
    assert np.abs(n(color) - f["color"]).max() <= 1e-4
    assert np.abs(n(out_all_map) - f["out_all_map"]).max() <= 1e-4
    assert np.array_equal(n(n_render), f["n_render"])
    assert np.array_equal(n(n_consider), f["n_consider"])
    assert np.array_equal(n(n_contrib), f["n_contrib_tile"])
    assert np.array_equal(n(out_observe), f["out_observe"])
    rb = orc.render_bwd(b["ranges"], b["point_list"], pre["means2D"], pre["conic_opacity"], col_np, am,
                        f["out_all_map"], f["final_T"], f["n_contrib"], cl_np, np.zeros(3, np.float32), n(ug["color"]),
                        n(ug["all_map"]), n(ug["plane_depth"]), W, H, cam.tanfovx, cam.tanfovy)
    assert _rel(n(means2D.grad), rb["dL_dmeans2D"][:, :2]) <= 1e-3
    assert _rel(n(means2D_abs.grad), rb["dL_dmeans2D_abs"]) <= 1e-3
    pb = orc.preprocess_bwd(n(g["means3D"]), pre["radii"], n(g["shs"]) if sh_mode else None, pre["clamped"],
                            n(g["scales"]), n(g["rotations"]), pre["cov3D"], n(cam.world_view_transform),
                            n(cam.full_proj_transform), n(cam.camera_center), W, H, cam.tanfovx, cam.tanfovy,
                            rb["dL_dmeans2D"], rb["dL_dconic_opacity"], rb["dL_dcolors"])
    # all_map is built in torch from the same leaves, so its autograd path adds to these leaves;
    # compare the opacity and SH/colour gradients, which only flow through the rasterizer ops
    assert _rel(n(leaf["opacities"].grad), pb["dL_dopacity"]) <= 1e-3
    if sh_mode:
        assert leaf["shs"].grad.shape == (P, 16, 3)
        assert _rel(n(leaf["shs"].grad), pb["dL_dsh"]) <= 1e-3
    else:
        assert mlp_rgb.grad.shape == (P, 3)
        assert _rel(n(mlp_rgb.grad), rb["dL_dcolors"]) <= 1e-3
    for k in ("means3D", "scales", "rotations"):
        assert leaf[k].grad is not None and torch.isfinite(leaf[k].grad).all()


def test_rasterizer_only_grads_match_oracle(orc):
    """all_map detached, so the leaves' gradients come from the two rasterizer ops alone."""
    import gs_scenes
    from diff_gaussian_rasterization import GaussianRasterizer
    P = 120_000
    g, cams = gs_scenes.make_scene(1, P=P, n_views=1)
    cam = cams[0]
    W, H = cam.image_width, cam.image_height
    rast = GaussianRasterizer(_settings(cam, bg=(0.1, 0.2, 0.3)))
    leaf = {k: g[k].to(DEV).requires_grad_(True) for k in ("means3D", "scales", "rotations", "opacities", "shs")}
    ca = _cuda_args()
    means2D, rgb, co, radii, depths = rast.preprocess_gaussians(leaf["means3D"], leaf["scales"], leaf["rotations"],
                                                                leaf["shs"], leaf["opacities"], ca)
    am = gs_scenes.build_all_map(g["means3D"], g["scales"], g["rotations"], cam).to(DEV)
    gx, gy = (W + 15) // 16, (H + 15) // 16
    cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
    m2abs = torch.zeros(P, 3, device=DEV, requires_grad=True)
    color, _, _, _, _, oam, opd = rast.render_gaussians(means2D, m2abs, co, rgb, am, depths, radii, cl, cl, ca)
    ug = gs_scenes.upstream_grads(cam)
    ((color * ug["color"].to(DEV)).sum() + (oam * ug["all_map"].to(DEV)).sum() +
     (opd * ug["plane_depth"].to(DEV)).sum()).backward()
    n = lambda t: t.detach().cpu().numpy()
    pre = orc.preprocess_fwd(n(g["means3D"]), n(g["scales"]), n(g["rotations"]), n(g["opacities"]), n(g["shs"]),
                             n(cam.world_view_transform), n(cam.full_proj_transform), n(cam.camera_center), W, H,
                             cam.tanfovx, cam.tanfovy)
    cl_np = np.ones(gx * gy, bool)
    b = orc.bin_and_sort(pre["radii"], pre["means2D"], pre["depths"], cl_np, W, H)
    bg = np.array([0.1, 0.2, 0.3], np.float32)
    f = orc.render_fwd(b["ranges"], b["point_list"], pre["means2D"], pre["rgb"], n(am), pre["conic_opacity"], cl_np, bg,
                       W, H, cam.tanfovx, cam.tanfovy)
    rb = orc.render_bwd(b["ranges"], b["point_list"], pre["means2D"], pre["conic_opacity"], pre["rgb"], n(am),
                        f["out_all_map"], f["final_T"], f["n_contrib"], cl_np, bg, n(ug["color"]), n(ug["all_map"]),
                        n(ug["plane_depth"]), W, H, cam.tanfovx, cam.tanfovy)
    pb = orc.preprocess_bwd(n(g["means3D"]), pre["radii"], n(g["shs"]), pre["clamped"], n(g["scales"]),
                            n(g["rotations"]), pre["cov3D"], n(cam.world_view_transform), n(cam.full_proj_transform),
                            n(cam.camera_center), W, H, cam.tanfovx, cam.tanfovy, rb["dL_dmeans2D"],
                            rb["dL_dconic_opacity"], rb["dL_dcolors"])
    for k, r in (("means3D", "dL_dmeans3D"), ("scales", "dL_dscales"), ("rotations", "dL_drotations"),
                 ("opacities", "dL_dopacity"), ("shs", "dL_dsh")):
        assert _rel(n(leaf[k].grad), pb[r]) <= 1e-3, k
    assert _rel(n(m2abs.grad), rb["dL_dmeans2D_abs"]) <= 1e-3


def test_empty_inputs_and_errors():
    import gs_scenes
    from diff_gaussian_rasterization import GaussianRasterizer
    cam = gs_scenes.make_scene(0, P=10)[1][0]
    rast = GaussianRasterizer(_settings(cam))
    z = lambda *s: torch.zeros(*s, device=DEV)
    m2, rgb, co, radii, depths = rast.preprocess_gaussians(z(0, 3), z(0, 3), z(0, 4), z(0, 3), z(0, 1), _cuda_args())
    assert m2.shape == (0, 2) and radii.shape == (0,)
    gx, gy = (cam.image_width + 15) // 16, (cam.image_height + 15) // 16
    cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
    out = rast.render_gaussians(m2, z(0, 3), co, rgb, z(0, 5), depths, radii, cl, cl, _cuda_args())
    assert out[0].shape == (3, cam.image_height, cam.image_width) and float(out[0].abs().max()) == 0.0
    assert rast.visible_filter(z(0, 3), z(0, 3), z(0, 4)).shape == (0,)
    with pytest.raises(RuntimeError, match="num_points, 3"):
        rast.preprocess_gaussians(z(5, 2), z(5, 3), z(5, 4), z(5, 3), z(5, 1), _cuda_args())
    with pytest.raises(RuntimeError, match="GPU tensor"):
        rast.preprocess_gaussians(torch.zeros(5, 3), z(5, 3), z(5, 4), z(5, 3), z(5, 1), _cuda_args())


def test_all_gaussians_behind_camera_renders_background():
    import gs_scenes
    from diff_gaussian_rasterization import GaussianRasterizer
    g, cams = gs_scenes.make_scene(0, P=1000)
    cam = cams[0]
    rast = GaussianRasterizer(_settings(cam, bg=(0.25, 0.5, 0.75)))
    means = g["means3D"].clone()
    means[:, 2] = -100.0  # camera sits at z=-30 looking towards +z
    m2, rgb, co, radii, depths = rast.preprocess_gaussians(means.to(DEV), g["scales"].to(DEV), g["rotations"].to(DEV),
                                                           g["shs"].to(DEV), g["opacities"].to(DEV), _cuda_args())
    assert int(radii.max()) == 0
    gx, gy = (cam.image_width + 15) // 16, (cam.image_height + 15) // 16
    cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
    color, n_render, *_ = rast.render_gaussians(m2, torch.zeros(1000, 3, device=DEV), co, rgb,
                                                torch.zeros(1000, 5, device=DEV), depths, radii, cl, cl, _cuda_args())
    assert int(n_render.sum()) == 0
    assert torch.allclose(color[:, 0, 0].cpu(), torch.tensor([0.25, 0.5, 0.75]))
    assert float((color - color[:, :1, :1]).abs().max()) == 0.0


@pytest.mark.parametrize("cfg,P,mask,geo", [(0, 40_000, False, True), (1, 100_000, True, True), (0, 20_000, False, False)])
def test_max_weight_depth_matches_oracle_and_changes_nothing_else(orc, cfg, P, mask, geo):
    """The additional per-pixel output (depth of the Gaussian with the largest blending weight) equals the oracle's
    bit for bit, and asking for it leaves every other output of render_gaussians as it is."""
    import gpu_harness as H
    import gs_scenes
    from diff_gaussian_rasterization import _C
    g, cams = gs_scenes.make_scene(cfg, P=P, n_views=1)
    cam = cams[0]
    W, Hh = cam.image_width, cam.image_height
    gx, gy = H.grid(W, Hh)
    cl = torch.ones(gy, gx, dtype=torch.bool)
    if mask:
        cl[::2, 1::3] = False
    o, gd = H.preprocess_fwd(g, cam)
    vm, cp = cam.world_view_transform.to(DEV), cam.camera_center.to(DEV)
    am = gs_scenes.build_all_map(gd["means3D"], gd["scales"], gd["rotations"], cam)

    def run(args):
        return _C.render_gaussians(torch.zeros(3, device=DEV), Hh, W, o["means2D"], o["depths"], o["radii"],
                                   o["conic_opacity"], o["rgb"], cl.to(DEV), vm, cp, cam.tanfovx, cam.tanfovy, am,
                                   geo, False, args)

    plain_args = {"stats_collector": {}}
    plain = run(plain_args)
    assert "max_weight_depth" not in plain_args["stats_collector"]
    args = {"stats_collector": {}, "max_weight_depth": True}
    out = run(args)
    got = args["stats_collector"]["max_weight_depth"]
    assert got.shape == (1, Hh, W)
    px = cl.repeat_interleave(16, 0).repeat_interleave(16, 1)[:Hh, :W].to(DEV)
    for a, b in zip(plain[1:8], out[1:8]):
        if a.dim() == 3:
            assert torch.equal(a[:, px], b[:, px])
        else:
            assert torch.equal(a, b)
    n = lambda t: t.detach().cpu().numpy()
    bins = orc.bin_and_sort(n(o["radii"]), n(o["means2D"]), n(o["depths"]), cl.numpy().reshape(-1), W, Hh)
    want = orc.max_weight_depth(bins["ranges"], bins["point_list"], n(o["means2D"]), n(o["conic_opacity"]),
                                n(o["depths"]), cl.numpy().reshape(-1), W, Hh)
    pxn = n(px)
    assert np.array_equal(n(got)[0][pxn], want[0][pxn])
    assert float(got[0][px].max()) > 0


@pytest.mark.parametrize("geo", [True, False])
def test_pixels_of_tiles_not_computed_locally_read_zero(geo):
    """The reference allocates its images zero-filled (rasterize_points.cu:303-307) and its kernel skips tiles that
    are not computed locally, so their pixels read 0; a caller may sum a loss over the whole image.  Same here, in
    all three images and in the additional depth image, however dirty the allocator's memory is."""
    import gs_scenes
    from diff_gaussian_rasterization import GaussianRasterizer
    g, cams = gs_scenes.make_scene(0, P=20_000, n_views=1)
    cam = cams[0]
    W, H = cam.image_width, cam.image_height
    gx, gy = (W + 15) // 16, (H + 15) // 16
    cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
    cl[::2, ::2] = False
    cl[-1, :] = False
    # leave NaNs behind in the caching allocator's free blocks
    junk = [torch.full((s, H, W), float("nan"), device=DEV) for s in (3, 5, 1, 1)]
    del junk
    rast = GaussianRasterizer(_settings(cam, render_geo=geo, bg=(0.3, 0.6, 0.9)))
    d = {k: g[k].to(DEV) for k in ("means3D", "scales", "rotations", "opacities", "shs")}
    args = _cuda_args()
    args["max_weight_depth"] = True
    means2D, rgb, co, radii, depths = rast.preprocess_gaussians(d["means3D"], d["scales"], d["rotations"], d["shs"],
                                                                d["opacities"], args)
    am = gs_scenes.build_all_map(d["means3D"], d["scales"], d["rotations"], cam)
    color, n_render, n_consider, n_contrib, obs, oam, opd = rast.render_gaussians(
        means2D, torch.zeros_like(d["means3D"]), co, rgb, am, depths, radii, cl, cl, args)
    mwd = args["stats_collector"]["max_weight_depth"]
    px = cl.repeat_interleave(16, 0).repeat_interleave(16, 1)[:H, :W]
    for name, img in (("color", color), ("all_map", oam), ("plane_depth", opd), ("max_weight_depth", mwd)):
        assert bool(torch.isfinite(img).all()), name
        assert float(img[:, ~px].abs().max()) == 0.0, name
    assert float(color[:, px].min()) > 0.0  # the local pixels carry at least the background
    assert int(n_consider.view(gy, gx)[~cl].abs().sum()) == 0 and int(n_contrib.view(gy, gx)[~cl].abs().sum()) == 0
    assert float((color * px).sum()) == float(color.sum())


def test_launching_ahead_of_the_instance_count_changes_no_result(orc):
    """With an expectation of the view's size, render_gaussians launches the list kernels and the blend without
    waiting for the instance count.  Whether the expectation holds (kernels ran ahead), is too small in instances
    or in list length (they turn into no-ops and the lists are built again), or is absent: same outputs and same
    gradients, bit for bit; the buffers of a call that ran ahead are laid out for its capacity."""
    import ctypes as C
    import gs_scenes
    import gsrast_native as gn
    from diff_gaussian_rasterization import _C
    import gpu_harness as H
    g, cams = gs_scenes.make_scene(1, P=150_000, n_views=1)
    cam = cams[0]
    W, Hh = cam.image_width, cam.image_height
    gx, gy = H.grid(W, Hh)
    o, gd = H.preprocess_fwd(g, cam)
    vm, cp = cam.world_view_transform.to(DEV), cam.camera_center.to(DEV)
    am = gs_scenes.build_all_map(gd["means3D"], gd["scales"], gd["rotations"], cam)
    cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
    bg = torch.tensor([0.2, 0.1, 0.3], device=DEV)
    ug = {k: v.to(DEV) for k, v in gs_scenes.upstream_grads(cam).items()}

    def run(expected_instances=0, expected_longest=0):
        args = {"stats_collector": {}}
        out, info = _C.render_gaussians_ex(bg, Hh, W, o["means2D"], o["depths"], o["radii"], o["conic_opacity"],
                                           o["rgb"], cl, vm, cp, cam.tanfovx, cam.tanfovy, am, True, False, args,
                                           expected_instances=expected_instances,
                                           expected_longest_list=expected_longest)
        R, geomB, binB, imgB = out[0], out[8], out[9], out[10]
        back = _C.render_gaussians_backward(bg, cam.tanfovx, cam.tanfovy, out[6], am, R, geomB, binB, imgB, cl,
                                            ug["color"], ug["all_map"], ug["plane_depth"], o["means2D"],
                                            o["conic_opacity"], o["rgb"], True, False, args,
                                            binning_capacity=info["binning_capacity"])
        off = [C.c_size_t() for _ in range(5)]
        gn.check(gn.lib.gs_binning_state_layout(info["binning_capacity"], W, Hh, *[C.byref(x) for x in off]), "layout")
        base = (binB.data_ptr() + 255) // 256 * 256 - binB.data_ptr()
        point_list = binB[base + off[0].value: base + off[0].value + 4 * R].view(torch.int32).clone()
        keys = binB[base + off[1].value: base + off[1].value + 8 * R].view(torch.int64).clone()
        return out, info, back, point_list, keys

    plain = run()
    R, longest = plain[0][0], plain[1]["longest_list"]
    assert not plain[1]["launched_ahead"] and plain[1]["binning_capacity"] == R and 0 < longest <= 2048
    n = lambda t: t.detach().cpu().numpy()
    want = orc.bin_and_sort(n(o["radii"]), n(o["means2D"]), n(o["depths"]), np.ones(gx * gy, bool), W, Hh)
    assert np.array_equal(H.np_u32(plain[3]), want["point_list"])
    cases = [("holds", R + 1000, 2048, True), ("exact", R, longest, True), ("default list length", 2 * R, 0, True),
             ("too few instances", R - 1, 2048, False), ("list too long", R + 1000, longest - 1, False)]
    for name, exp_n, exp_l, ahead in cases:
        got = run(exp_n, exp_l)
        assert got[1]["launched_ahead"] == ahead, name
        assert got[1]["binning_capacity"] == (exp_n if ahead else R), name
        assert got[1]["longest_list"] == longest and got[0][0] == R, name
        for a, b in zip(plain[0][1:8], got[0][1:8]):
            assert torch.equal(a, b), name
        for a, b in zip(plain[2], got[2]):
            assert torch.equal(a, b), name
        assert torch.equal(plain[3], got[3]) and torch.equal(plain[4], got[4]), name


def test_the_operator_launches_ahead_from_the_second_view_on():
    """GaussianRasterizer remembers what the last view of a shape needed and launches the next one ahead; the
    gradients of the leaves are the same bits as on the first, ordinary call."""
    import gs_scenes
    import diff_gaussian_rasterization as dgr
    g, cams = gs_scenes.make_scene(0, P=25_000, n_views=1)
    cam = cams[0]
    W, H = cam.image_width, cam.image_height
    gx, gy = (W + 15) // 16, (H + 15) // 16
    cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
    ug = {k: v.to(DEV) for k, v in gs_scenes.upstream_grads(cam).items()}
    am = gs_scenes.build_all_map(g["means3D"], g["scales"], g["rotations"], cam).to(DEV)
    dgr._expectations.clear()

    def run():
        rast = dgr.GaussianRasterizer(_settings(cam))
        leaf = {k: g[k].to(DEV).requires_grad_(True) for k in ("means3D", "scales", "rotations", "opacities", "shs")}
        args = _cuda_args()
        means2D, rgb, co, radii, depths = rast.preprocess_gaussians(
            leaf["means3D"], leaf["scales"], leaf["rotations"], leaf["shs"], leaf["opacities"], args)
        m2abs = torch.zeros_like(leaf["means3D"], requires_grad=True) + 0
        color, n_render, n_consider, n_contrib, obs, oam, opd = rast.render_gaussians(
            means2D, m2abs, co, rgb, am, depths, radii, cl, cl, args)
        torch.autograd.backward([color, oam, opd], [ug["color"], ug["all_map"], ug["plane_depth"]])
        return [color, n_render, n_consider, n_contrib, obs, oam, opd] + [leaf[k].grad for k in sorted(leaf)]

    first = run()
    key = (H, W, torch.device(DEV))
    assert key in dgr._expectations and dgr._expectation(key)[0] > dgr._expectations[key][0]
    for _ in range(2):
        again = run()
        for a, b in zip(first, again):
            assert torch.equal(a, b)
    # the table of expectations stays small whatever sizes come by
    for k in range(3 * dgr._MAX_EXPECTATIONS):
        dgr._remember((100 + k, 100, torch.device(DEV)), 1000, 100)
    assert len(dgr._expectations) == dgr._MAX_EXPECTATIONS and (100, 100, torch.device(DEV)) not in dgr._expectations
    dgr._expectations.clear()


def test_debug_mode_gives_the_same_results_by_every_route():
    """debug=True makes every stage wait for its kernels and report their errors (and check the radix sort's
    status word); results are those of the normal mode bit for bit, whichever way the per-tile lists are built."""
    import gs_scenes
    import gsrast_native as gn
    from diff_gaussian_rasterization import GaussianRasterizer
    g, cams = gs_scenes.make_scene(0, P=30_000, n_views=1)
    cam = cams[0]
    W, H = cam.image_width, cam.image_height
    gx, gy = (W + 15) // 16, (H + 15) // 16
    cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
    ug = {k: v.to(DEV) for k, v in gs_scenes.upstream_grads(cam).items()}

    def run(debug, limits=None):
        rast = GaussianRasterizer(_settings(cam)._replace(debug=debug))
        leaf = {k: g[k].to(DEV).requires_grad_(True) for k in ("means3D", "scales", "rotations", "opacities", "shs")}
        args = _cuda_args()
        if limits is not None:
            args["tile_sort_limits"] = limits
        means2D, rgb, co, radii, depths = rast.preprocess_gaussians(
            leaf["means3D"], leaf["scales"], leaf["rotations"], leaf["shs"], leaf["opacities"], args)
        am = gs_scenes.build_all_map(leaf["means3D"], leaf["scales"], leaf["rotations"], cam)
        m2abs = torch.zeros_like(leaf["means3D"], requires_grad=True) + 0
        color, n_render, n_consider, n_contrib, obs, oam, opd = rast.render_gaussians(
            means2D, m2abs, co, rgb, am, depths, radii, cl, cl, args)
        torch.autograd.backward([color, oam, opd], [ug["color"], ug["all_map"], ug["plane_depth"]])
        return [color, n_render, n_consider, n_contrib, obs, oam] + [leaf[k].grad for k in sorted(leaf)]

    base = run(False)
    for limits in [(-1, -1), (0, 0), (40, 0), (100, 128)]:
        got = run(True, limits)
        for i, (a, b) in enumerate(zip(base[:6], got[:6])):
            assert torch.equal(a, b), (limits, i)
        for i, (a, b) in enumerate(zip(base[6:], got[6:])):
            assert float((a - b).norm()) <= 1e-5 * float(a.norm()) + 1e-12, (limits, i)
    # the route is a per-call option: the call after a forced radix route takes the default route again, and a
    # call from another thread in between is not affected either (the library keeps no such setting)
    import threading
    seen = {}
    t = threading.Thread(target=lambda: seen.setdefault("other", run(False)))
    t.start()
    t.join()
    for a, b in zip(base[:6], seen["other"][:6]):
        assert torch.equal(a, b)


@pytest.mark.parametrize("geo", [True, False])
def test_records_written_by_the_producers_give_the_same_results(geo):
    """From the second view of an image size on, preprocess_gaussians starts the blend kernels' operand records and
    build_all_map(..., blend_records_of=means2D) finishes them, so that render_gaussians packs nothing.  Outputs and
    gradients are the bits of the first view (whose records the library packed); a tensor that is replaced or
    modified on the way makes render_gaussians fall back to packing, again with the same bits."""
    import gs_scenes
    import diff_gaussian_rasterization as dgr
    import gsrast_native as gn
    g, cams = gs_scenes.make_scene(1, P=40_000, n_views=1)
    cam = cams[0]
    W, H = cam.image_width, cam.image_height
    gx, gy = (W + 15) // 16, (H + 15) // 16
    cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
    ug = {k: v.to(DEV) for k, v in gs_scenes.upstream_grads(cam).items()}
    dgr._expectations.clear()
    dgr._linked_all_map_seen[0] = False

    def run(disturb=None):
        rs = _settings(cam, render_geo=geo)
        rast = dgr.GaussianRasterizer(rs)
        leaf = {k: g[k].to(DEV).requires_grad_(True) for k in ("means3D", "scales", "rotations", "opacities", "shs")}
        args = _cuda_args()
        means2D, rgb, co, radii, depths = rast.preprocess_gaussians(
            leaf["means3D"], leaf["scales"], leaf["rotations"], leaf["shs"], leaf["opacities"], args)
        started = getattr(means2D, "_gs_blend", None) is not None
        am = dgr.build_all_map(leaf["means3D"], leaf["scales"], leaf["rotations"], rs.viewmatrix, rs.campos,
                               blend_records_of=means2D)
        if disturb == "replace":
            am = am * 1.0  # the same values in another tensor
        elif disturb == "modify":
            with torch.no_grad():
                rgb.mul_(1.0)  # (an in-place operation on one of the tensors the records were written from)
        m2abs = torch.zeros_like(leaf["means3D"], requires_grad=True) + 0
        gn.stage_timing(True)
        color, n_render, n_consider, n_contrib, obs, oam, opd = rast.render_gaussians(
            means2D, m2abs, co, rgb, am, depths, radii, cl, cl, args)
        torch.autograd.backward([color, oam, opd] if geo else [color],
                                [ug["color"], ug["all_map"], ug["plane_depth"]] if geo else [ug["color"]])
        torch.cuda.synchronize()
        gn.stage_timing(False)
        packed_by_library = gn.stage_timing_collect().get("pack_operands", (0.0, 0))[1] > 0
        outs = [color, n_render, n_consider, n_contrib, obs, oam, opd] + [leaf[k].grad for k in sorted(leaf)]
        return started, packed_by_library, outs

    started, packed_by_library, first = run()
    assert not started and packed_by_library  # nothing is known about this image size yet
    used = 0
    for disturb in (None, None, "replace", None, None, "modify", None, None):
        started, packed_by_library, again = run(disturb)
        if disturb == "modify" or not started:
            assert packed_by_library, disturb
        elif disturb is None:
            assert not packed_by_library
            used += 1
        elif disturb == "replace":
            # (with no geometry channels to render, the all_map tensor is not part of the records)
            assert packed_by_library == geo
        for a, b in zip(first, again):
            assert torch.equal(a, b), disturb
    assert used >= 3
    dgr._expectations.clear()
    dgr._linked_all_map_seen[0] = False


@pytest.mark.parametrize("poison", [False, True])
def test_packed_and_gathered_operands_give_the_same_results(poison):
    """The forward call packs the blend kernels' operands into one record per Gaussian when the view has more than
    0.8 instances per Gaussian, and lets both blend kernels gather them from the caller's arrays otherwise.  The
    same Gaussians with and without a crowd of Gaussians behind the camera (which adds no instance and tips the
    decision) must render and differentiate to the same bits; so must a view in which some Gaussians carry NaN or
    infinite colours and geometry channels (NaNs in the same places, the same bits everywhere else)."""
    import gs_scenes
    from diff_gaussian_rasterization import GaussianRasterizer
    g, cams = gs_scenes.make_scene(1, P=40_000, n_views=1)
    cam = cams[0]
    W, H = cam.image_width, cam.image_height
    gx, gy = (W + 15) // 16, (H + 15) // 16
    cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
    ug = {k: v.to(DEV) for k, v in gs_scenes.upstream_grads(cam).items()}
    P = g["means3D"].shape[0]

    def run(extra):
        h = {k: g[k] for k in ("means3D", "scales", "rotations", "opacities", "shs")}
        if extra:
            # behind the camera: culled by the preprocess, radius 0, no instance
            eye = cam.camera_center.reshape(1, 3).cpu()
            look = torch.zeros(1, 3) - eye
            behind = eye - 5.0 * look / look.norm() + 0.1 * torch.randn(extra, 3, generator=torch.Generator().manual_seed(1))
            h = {"means3D": torch.cat([h["means3D"], behind]),
                 "scales": torch.cat([h["scales"], h["scales"][:1].expand(extra, -1)]),
                 "rotations": torch.cat([h["rotations"], h["rotations"][:1].expand(extra, -1)]),
                 "opacities": torch.cat([h["opacities"], h["opacities"][:1].expand(extra, -1)]),
                 "shs": torch.cat([h["shs"], h["shs"][:1].expand(extra, -1, -1)])}
        rast = GaussianRasterizer(_settings(cam))
        leaf = {k: v.to(DEV).requires_grad_(True) for k, v in h.items()}
        args = _cuda_args()
        means2D, rgb, co, radii, depths = rast.preprocess_gaussians(
            leaf["means3D"], leaf["scales"], leaf["rotations"], leaf["shs"], leaf["opacities"], args)
        assert int((radii[P:] > 0).sum()) == 0
        am = gs_scenes.build_all_map(leaf["means3D"], leaf["scales"], leaf["rotations"], cam)
        if poison:
            vis = torch.nonzero(radii[:P] > 0)[:, 0]
            pick = vis[torch.randperm(vis.numel(), generator=torch.Generator().manual_seed(3))[:40].to(vis.device)]
            rgb = rgb.detach().clone()
            am = am.detach().clone()
            rgb[pick[:10], 0] = float("nan")
            rgb[pick[10:20], 2] = float("inf")
            am[pick[20:30], 1] = float("nan")
            am[pick[30:40], 4] = float("-inf")
            rgb.requires_grad_(True)
            am.requires_grad_(True)
        m2abs = torch.zeros_like(leaf["means3D"], requires_grad=True) + 0
        color, n_render, n_consider, n_contrib, obs, oam, opd = rast.render_gaussians(
            means2D, m2abs, co, rgb, am, depths, radii, cl, cl, args)
        torch.autograd.backward([color, oam, opd], [ug["color"], ug["all_map"], ug["plane_depth"]])
        R = int(n_render.sum())
        return R, [color, n_render, n_consider, n_contrib, obs[:P], oam, opd] + [leaf[k].grad[:P] for k in sorted(leaf)]

    R, packed = run(0)
    assert R * 5 > P * 4, "the plain scene is meant to take the packed route"
    extra = 2 * R  # more than R / 0.8 - P
    R2, gathered = run(extra)
    assert R2 == R and R2 * 5 <= (P + extra) * 4
    for a, b in zip(packed, gathered):
        if a.is_floating_point():
            assert torch.equal(torch.isnan(a), torch.isnan(b))
            assert torch.equal(torch.nan_to_num(a, nan=0.0), torch.nan_to_num(b, nan=0.0))
        else:
            assert torch.equal(a, b)
    if poison:
        assert bool(torch.isnan(packed[0]).any()) and float(torch.isnan(packed[0]).float().mean()) < 0.2


def test_side_stream_gives_the_same_results():
    """Everything runs on the caller's current stream: the same step on a side stream (default priority), with
    other work in flight on the default stream, gives the same results, bit for bit."""
    import gs_scenes
    from diff_gaussian_rasterization import GaussianRasterizer
    g, cams = gs_scenes.make_scene(1, P=120_000, n_views=1)
    cam = cams[0]
    W, H = cam.image_width, cam.image_height
    gx, gy = (W + 15) // 16, (H + 15) // 16
    cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
    ug = {k: v.to(DEV) for k, v in gs_scenes.upstream_grads(cam).items()}
    dev = {k: g[k].to(DEV) for k in ("means3D", "scales", "rotations", "opacities", "shs")}
    torch.cuda.synchronize()

    def run():
        rast = GaussianRasterizer(_settings(cam))
        leaf = {k: v.clone().requires_grad_(True) for k, v in dev.items()}
        args = _cuda_args()
        means2D, rgb, co, radii, depths = rast.preprocess_gaussians(
            leaf["means3D"], leaf["scales"], leaf["rotations"], leaf["shs"], leaf["opacities"], args)
        am = gs_scenes.build_all_map(leaf["means3D"], leaf["scales"], leaf["rotations"], cam)
        m2abs = torch.zeros_like(leaf["means3D"], requires_grad=True) + 0
        color, n_render, n_consider, n_contrib, obs, oam, opd = rast.render_gaussians(
            means2D, m2abs, co, rgb, am, depths, radii, cl, cl, args)
        torch.autograd.backward([color, oam, opd], [ug["color"], ug["all_map"], ug["plane_depth"]])
        return [color, n_render, n_consider, n_contrib, obs, oam] + [leaf[k].grad for k in sorted(leaf)]

    base = run()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    busy = torch.randn(4096, 4096, device=DEV)
    with torch.cuda.stream(side):
        for _ in range(3):
            busy = busy @ busy * 1e-3  # keeps the default stream's queue independent of the side stream's
        got = run()
    side.synchronize()
    torch.cuda.synchronize()
    # gradients too: every sum of the backward pass is taken in a fixed order (no float atomics anywhere)
    for i, (a, b) in enumerate(zip(base, got)):
        assert torch.equal(a, b), i


def test_views_in_flight_on_two_streams_give_the_same_results():
    """A batch's views alternate between two streams (default priority), so that one view's bandwidth-bound
    stages run beside the other's blend kernels: every view's outputs and gradients are the bits of the same
    view rendered alone."""
    import gs_scenes
    from diff_gaussian_rasterization import GaussianRasterizer
    g, cams = gs_scenes.make_scene(2, P=200_000, n_views=4)
    W, H = cams[0].image_width, cams[0].image_height
    gx, gy = (W + 15) // 16, (H + 15) // 16
    cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
    ugs = [{k: v.to(DEV) for k, v in gs_scenes.upstream_grads(c, seed=i).items()} for i, c in enumerate(cams)]
    dev = {k: g[k].to(DEV) for k in ("means3D", "scales", "rotations", "opacities", "shs")}
    ams = [gs_scenes.build_all_map(g["means3D"], g["scales"], g["rotations"], c).to(DEV) for c in cams]
    torch.cuda.synchronize()

    def run(v):
        rast = GaussianRasterizer(_settings(cams[v]))
        leaf = {k: t.clone().requires_grad_(True) for k, t in dev.items()}
        args = _cuda_args()
        means2D, rgb, co, radii, depths = rast.preprocess_gaussians(
            leaf["means3D"], leaf["scales"], leaf["rotations"], leaf["shs"], leaf["opacities"], args)
        m2abs = torch.zeros_like(leaf["means3D"], requires_grad=True) + 0
        color, n_render, n_consider, n_contrib, obs, oam, opd = rast.render_gaussians(
            means2D, m2abs, co, rgb, ams[v], depths, radii, cl, cl, args)
        torch.autograd.backward([color, oam, opd], [ugs[v]["color"], ugs[v]["all_map"], ugs[v]["plane_depth"]])
        return [color, n_render, n_consider, n_contrib, obs, oam, opd] + [leaf[k].grad for k in sorted(leaf)]

    alone = []
    for v in range(len(cams)):
        alone.append(run(v))
        torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for s in streams:
        s.wait_stream(torch.cuda.current_stream())
    together = []
    for rep in range(3):  # twelve views, at most two in flight
        for v in range(len(cams)):
            with torch.cuda.stream(streams[v % 2]):
                together.append((v, run(v)))
    for s in streams:
        s.synchronize()
    for v, got in together:
        for i, (a, b) in enumerate(zip(alone[v], got)):
            assert torch.equal(a, b), (v, i)


def test_per_tile_debug_log_is_written_like_the_reference(tmp_path):
    """cuda_args with mode == "train", zhx_debug == "True" and iteration % log_interval == 1 make the forward call
    append the reference's per-tile log (cuda_rasterizer/rasterizer_impl.cu:764-842): one line per tile with a
    non-empty list and one line of totals, in its file name and format; other iterations write nothing."""
    import re
    import gs_scenes
    from diff_gaussian_rasterization import GaussianRasterizer
    g, cams = gs_scenes.make_scene(0, P=20_000, n_views=1)
    cam = cams[0]
    W, H = cam.image_width, cam.image_height
    gx, gy = (W + 15) // 16, (H + 15) // 16
    rast = GaussianRasterizer(_settings(cam))
    d = {k: g[k].to(DEV) for k in ("means3D", "scales", "rotations", "opacities", "shs")}
    cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
    am = gs_scenes.build_all_map(g["means3D"], g["scales"], g["rotations"], cam).to(DEV)

    def run(iteration):
        args = _cuda_args()
        args.update(zhx_debug="True", iteration=str(iteration), log_interval="10", log_folder=str(tmp_path))
        means2D, rgb, co, radii, depths = rast.preprocess_gaussians(d["means3D"], d["scales"], d["rotations"],
                                                                    d["shs"], d["opacities"], args)
        m2abs = torch.zeros_like(d["means3D"])
        return rast.render_gaussians(means2D, m2abs, co, rgb, am, depths, radii, cl, cl, args)

    path = tmp_path / "n_contrib_ws=1_rk=0.log"
    run(2)
    assert not path.exists()
    color, n_render, n_consider, n_contrib, *_ = run(11)
    lines = path.read_text().splitlines()
    nr, nc, n2 = (t.cpu().numpy().astype(np.int64) for t in (n_render, n_consider, n_contrib))
    busy = np.nonzero(nr > 0)[0]
    assert len(lines) == len(busy) + 1 and len(busy) > 100
    pat = re.compile(r"iteration: 11, tile: \((\d+), (\d+)\), range: \((\d+), (\d+)\), num_rendered_this_tile: (\d+), "
                     r"n_considered_per_pixel: ([\d.]+), n_contrib2loss_per_pixel: ([\d.]+), contrib2loss_ratio: ([\d.]+)$")
    ends = np.cumsum(nr)
    for line, t in zip(lines, busy):
        m = pat.match(line)
        assert m, line
        ty, tx, end, begin, n = (int(m.group(i)) for i in range(1, 6))
        assert (ty, tx) == (t // gx, t % gx) and n == nr[t] and end == ends[t] and begin == ends[t] - nr[t]
        assert abs(float(m.group(6)) - nc[t] / 256.0) < 1e-5 and abs(float(m.group(7)) - n2[t] / 256.0) < 1e-5
    assert lines[-1].startswith("iteration: 11, global_rank: 0, world_size: 1, num_tiles: %d, num_pixels: %d, "
                                "num_rendered: %d," % (len(busy), 256 * len(busy), nr.sum()))
    run(21)
    assert len(path.read_text().splitlines()) == 2 * (len(busy) + 1)  # appended, like the reference
