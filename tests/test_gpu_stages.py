"""GPU parity of every stage of the rasterizer against the CPU oracle, through
the C ABI.  Integer and index outputs must be identical; images within 1e-4
absolute; gradients within 1e-3 relative L2."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

IMG_TOL = 1e-4
GRAD_TOL = 1e-3


@pytest.fixture(scope="module")
def H():
    import gpu_harness
    assert torch.cuda.is_available()
    return gpu_harness


def _scene(cfg, P):
    import gs_scenes
    g, cams = gs_scenes.make_scene(cfg, P=P, n_views=1)
    return g, cams[0]


CASES = [(0, 50_000), (1, 200_000), (3, 60_000)]


@pytest.mark.parametrize("cfg,P", CASES)
@pytest.mark.parametrize("sh_mode", [True, False])
def test_preprocess_forward(H, orc, cfg, P, sh_mode):
    g, cam = _scene(cfg, P)
    got, _ = H.preprocess_fwd(g, cam, sh_mode=sh_mode)
    ref = H.oracle_preprocess(orc, g, cam, sh_mode=sh_mode)
    assert np.array_equal(got["radii"].cpu().numpy(), ref["radii"])
    assert np.array_equal(H.np_u32(got["tiles_touched"]), ref["tiles_touched"])
    # depth feeds the sort key: bits must agree
    assert np.array_equal(H.np_u32(got["depths"].view(torch.int32)), ref["depths"].view(np.uint32))
    assert np.array_equal(got["clamped"].cpu().numpy(), ref["clamped"])
    for k in ("means2D", "cov3D", "conic_opacity", "rgb"):
        a, b = got[k].cpu().numpy(), ref[k]
        assert np.array_equal(a, b), f"{k}: max abs diff {np.abs(a - b).max()}"
    assert (ref["radii"] > 0).any() and (ref["radii"] == 0).any() or cfg == 0


@pytest.mark.parametrize("degree,M", [(0, 16), (1, 16), (2, 16), (3, 16), (0, 1), (1, 4), (2, 9), (1, 9)])
@pytest.mark.parametrize("P", [1, 63, 64, 65, 33_333])
def test_preprocess_colours_at_every_degree_and_row_length(H, orc, degree, M, P):
    """Active SH degrees below the stored one (the caller raises the degree as training goes on), rows shorter than
    16 coefficients, and Gaussian counts that end inside a wave: colours and clamp flags equal the oracle's bits."""
    g, cam = _scene(0, P)
    g = dict(g)
    g["shs"] = g["shs"][:, :M].contiguous()
    got, _ = H.preprocess_fwd(g, cam, sh_mode=True, sh_degree=degree)
    ref = H.oracle_preprocess(orc, g, cam, sh_mode=True, sh_degree=degree)
    assert np.array_equal(got["radii"].cpu().numpy(), ref["radii"])
    assert np.array_equal(got["clamped"].cpu().numpy(), ref["clamped"])
    for k in ("means2D", "cov3D", "conic_opacity", "rgb"):
        a, b = got[k].cpu().numpy(), ref[k]
        assert np.array_equal(a, b), f"{k}: max abs diff {np.abs(a - b).max()}"


@pytest.mark.parametrize("cfg,P", CASES)
def test_visible_filter_and_mark_visible(H, orc, cfg, P):
    import ctypes as C
    g, cam = _scene(cfg, P)
    gd = {k: H.dev(v) for k, v in g.items() if torch.is_tensor(v)}
    V, PM = H.dev(cam.world_view_transform), H.dev(cam.full_proj_transform)
    W, Hh = cam.image_width, cam.image_height
    radii = torch.full((P,), 9, dtype=torch.int32, device=H.DEV)
    H.gn.check(H.lib.gs_visible_filter(P, 0, W, Hh, H.ptr(gd["means3D"]), H.ptr(gd["scales"]), 1.0,
                                       H.ptr(gd["rotations"]), None, H.ptr(V), H.ptr(PM), cam.tanfovx, cam.tanfovy, 0,
                                       H.ptr(radii), 1, H.stream()), "gs_visible_filter")
    n = lambda t: t.numpy()
    ref = orc.visible_filter(n(g["means3D"]), n(g["scales"]), n(g["rotations"]), None, n(cam.world_view_transform),
                             n(cam.full_proj_transform), W, Hh, cam.tanfovx, cam.tanfovy)
    assert np.array_equal(radii.cpu().numpy(), ref)
    # with a precomputed covariance instead of scale/rotation
    pre = H.oracle_preprocess(orc, g, cam, sh_mode=False)
    cov = H.dev(pre["cov3D"])
    radii2 = torch.full((P,), 9, dtype=torch.int32, device=H.DEV)
    H.gn.check(H.lib.gs_visible_filter(P, 0, W, Hh, H.ptr(gd["means3D"]), None, 1.0, None, H.ptr(cov), H.ptr(V),
                                       H.ptr(PM), cam.tanfovx, cam.tanfovy, 0, H.ptr(radii2), 1, H.stream()),
               "gs_visible_filter")
    ref2 = orc.visible_filter(n(g["means3D"]), None, None, pre["cov3D"], n(cam.world_view_transform),
                              n(cam.full_proj_transform), W, Hh, cam.tanfovx, cam.tanfovy)
    assert np.array_equal(radii2.cpu().numpy(), ref2)
    present = torch.full((P,), 7, dtype=torch.uint8, device=H.DEV)
    H.gn.check(H.lib.gs_mark_visible(P, H.ptr(gd["means3D"]), H.ptr(V), H.ptr(PM), H.ptr(present), H.stream()),
               "gs_mark_visible")
    assert np.array_equal(present.cpu().numpy().astype(bool),
                          orc.mark_visible(n(g["means3D"]), n(cam.world_view_transform), n(cam.full_proj_transform)))


def _mask(kind, gx, gy):
    cl = np.ones((gy, gx), bool)
    if kind == "rows":
        cl[: gy // 3] = False
    elif kind == "checker":
        cl[::2, ::2] = False
    return cl.ravel()


@pytest.mark.parametrize("cfg,P,mask", [(0, 50_000, "all"), (1, 200_000, "all"), (1, 100_000, "rows"),
                                        (3, 60_000, "checker")])
def test_binning_stages(H, orc, cfg, P, mask):
    g, cam = _scene(cfg, P)
    W, Hh = cam.image_width, cam.image_height
    gx, gy = H.grid(W, Hh)
    pre = H.oracle_preprocess(orc, g, cam)
    cl = _mask(mask, gx, gy)
    ref = orc.bin_and_sort(pre["radii"], pre["means2D"], pre["depths"], cl, W, Hh)
    got = H.bin_stages(H.dev(pre["radii"]), H.dev(pre["means2D"]), H.dev(pre["depths"]), H.dev(cl), W, Hh)
    assert got["num_rendered"] == ref["num_rendered"] > 0
    for k in ("tiles_touched", "point_offsets", "keys_unsorted", "vals_unsorted", "keys", "point_list", "ranges"):
        assert np.array_equal(got[k], ref[k]), k


def _render_inputs(H, orc, cfg, P, mask="all"):
    import gs_scenes
    g, cam = _scene(cfg, P)
    W, Hh = cam.image_width, cam.image_height
    gx, gy = H.grid(W, Hh)
    pre = H.oracle_preprocess(orc, g, cam)
    cl = _mask(mask, gx, gy)
    b = orc.bin_and_sort(pre["radii"], pre["means2D"], pre["depths"], cl, W, Hh)
    am = gs_scenes.build_all_map(g["means3D"], g["scales"], g["rotations"], cam).numpy()
    return g, cam, pre, cl, b, am


@pytest.mark.parametrize("cfg,P,mask,geo,bgv", [(0, 50_000, "all", True, 0.0), (1, 200_000, "all", True, 0.3),
                                                (1, 100_000, "rows", True, 0.0), (3, 60_000, "all", False, 1.0),
                                                (3, 60_000, "checker", True, 0.5)])
def test_render_forward(H, orc, cfg, P, mask, geo, bgv):
    g, cam, pre, cl, b, am = _render_inputs(H, orc, cfg, P, mask)
    W, Hh = cam.image_width, cam.image_height
    bg = np.array([bgv, 0.5 * bgv, 1.0 - bgv], np.float32)
    ref = orc.render_fwd(b["ranges"], b["point_list"], pre["means2D"], pre["rgb"], am, pre["conic_opacity"], cl, bg, W,
                         Hh, cam.tanfovx, cam.tanfovy, render_geo=geo)
    got = H.render_fwd(P, W, Hh, cam.tanfovx, cam.tanfovy, H.as_u32(b["ranges"]), H.as_u32(b["point_list"]),
                       H.dev(pre["means2D"]), H.dev(pre["rgb"]), H.dev(am), H.dev(pre["conic_opacity"]), H.dev(cl),
                       H.dev(bg), render_geo=geo)
    gx, gy = H.grid(W, Hh)
    # the per-pixel state of tiles that are not computed locally is left untouched by both sides
    pix_local = np.repeat(np.repeat(cl.reshape(gy, gx), 16, 0), 16, 1)[:Hh, :W]
    for k in ("n_contrib", "n_contrib2loss"):
        assert np.array_equal(H.np_u32(got[k])[pix_local], ref[k][pix_local]), k
    assert np.array_equal(got["out_observe"].cpu().numpy(), ref["out_observe"])
    for k in ("n_render", "n_consider", "n_contrib_tile"):
        assert np.array_equal(got[k].cpu().numpy(), ref[k]), k
    # the transmittance decides the contributor counts: the same bits
    assert np.array_equal(got["final_T"].cpu().numpy()[pix_local], ref["final_T"][pix_local])
    # The images are the oracle's bit for bit (same operation order, explicit FMAs, the same exp); the plane
    # depth is a quotient formed in double precision on both sides, compared element by element.
    keys = ("color", "out_all_map", "out_plane_depth") if geo else ("color",)
    for k in keys:
        a, r = got[k].cpu().numpy()[:, pix_local], ref[k][:, pix_local]
        assert np.array_equal(np.isnan(a), np.isnan(r)), k
        ok = ~np.isnan(r)
        assert np.array_equal(a[ok], r[ok]), f"{k}: {np.abs(a[ok] - r[ok]).max()}"
        # pixels of tiles that are not computed locally read zero, as the reference's zero-filled images do
        # (rasterize_points.cu:303-307); the harness pre-fills every output with 55
        assert float(np.abs(got[k].cpu().numpy()[:, ~pix_local]).max(initial=0.0)) == 0.0, k
    if not geo:
        assert float(got["out_all_map"].abs().max()) == 0.0 and float(got["out_plane_depth"].abs().max()) == 0.0


@pytest.mark.parametrize("cfg,P,mask,geo", [(0, 50_000, "all", True), (1, 200_000, "all", True),
                                            (1, 100_000, "rows", True), (3, 60_000, "all", False)])
def test_render_backward(H, orc, cfg, P, mask, geo):
    import gs_scenes
    g, cam, pre, cl, b, am = _render_inputs(H, orc, cfg, P, mask)
    W, Hh = cam.image_width, cam.image_height
    bg = np.array([0.2, 0.4, 0.6], np.float32)
    f = orc.render_fwd(b["ranges"], b["point_list"], pre["means2D"], pre["rgb"], am, pre["conic_opacity"], cl, bg, W,
                       Hh, cam.tanfovx, cam.tanfovy, render_geo=geo)
    ug = gs_scenes.upstream_grads(cam)
    gpix, gmap, gdep = ug["color"].numpy(), ug["all_map"].numpy(), ug["plane_depth"].numpy()
    ref = orc.render_bwd(b["ranges"], b["point_list"], pre["means2D"], pre["conic_opacity"], pre["rgb"], am,
                         f["out_all_map"], f["final_T"], f["n_contrib"], cl, bg, gpix, gmap, gdep, W, Hh, cam.tanfovx,
                         cam.tanfovy, render_geo=geo)
    got = H.render_bwd(P, W, Hh, cam.tanfovx, cam.tanfovy, H.dev(bg), H.as_u32(b["ranges"]), H.as_u32(b["point_list"]),
                       H.dev(pre["means2D"]), H.dev(pre["conic_opacity"]), H.dev(pre["rgb"]), H.dev(am),
                       H.dev(f["out_all_map"]), H.dev(f["final_T"]), H.as_u32(f["n_contrib"]), H.dev(cl), H.dev(gpix),
                       H.dev(gmap), H.dev(gdep), H.as_u32(b["emission_sorted"]), H.as_u32(b["point_offsets"]),
                       render_geo=geo)
    pairs = [("dL_dmeans2D", ref["dL_dmeans2D"][:, :2]), ("dL_dmeans2D_abs", ref["dL_dmeans2D_abs"]),
             ("dL_dconic_opacity", ref["dL_dconic_opacity"]), ("dL_dcolors", ref["dL_dcolors"])]
    if geo:
        pairs.append(("dL_dall_map", ref["dL_dall_map"]))
    for k, r in pairs:
        a = got[k].cpu().numpy()
        assert np.isfinite(a).all(), k
        assert H.rel_l2(a, r) <= GRAD_TOL, f"{k}: rel L2 {H.rel_l2(a, r)}"
        # ... and row by row, so that a wrong gradient of a Gaussian with a small one cannot hide behind the
        # large ones: each element within 1e-3 of its own size plus 1e-5 of the tensor's largest
        worst = np.abs(a - r) - (GRAD_TOL * np.abs(r) + 1e-5 * np.abs(r).max())
        assert worst.max() <= 0.0, f"{k}: element {np.unravel_index(worst.argmax(), worst.shape)} off by {worst.max()}"
    a = got["dL_dmeans2D_abs"].cpu().numpy()
    assert (a[:, :2] + 1e-3 * np.abs(a[:, :2]) + 1e-6 >= np.abs(got["dL_dmeans2D"].cpu().numpy())).all()
    assert (a[:, 2] == 0).all()
    if not geo:
        assert float(got["dL_dall_map"].abs().max()) == 0.0


@pytest.mark.parametrize("cfg,P", CASES)
@pytest.mark.parametrize("sh_mode", [True, False, "saved"])
def test_preprocess_backward(H, orc, cfg, P, sh_mode):
    """sh_mode "saved": the backward call gets the forward call's derivative of the colours with respect to the
    view direction instead of the coefficients (shs = NULL): the same bits as with the coefficients."""
    saved = sh_mode == "saved"
    sh_mode = bool(sh_mode)
    g, cam = _scene(cfg, P)
    W, Hh = cam.image_width, cam.image_height
    pre = H.oracle_preprocess(orc, g, cam, sh_mode=sh_mode)
    gen = torch.Generator().manual_seed(5)
    g2 = torch.randn(P, 2, generator=gen).numpy()
    gco = torch.randn(P, 4, generator=gen).numpy()
    gcol = torch.randn(P, 3, generator=gen).numpy()
    n = lambda t: t.numpy()
    ref = orc.preprocess_bwd(n(g["means3D"]), pre["radii"], n(g["shs"]) if sh_mode else None, pre["clamped"],
                             n(g["scales"]), n(g["rotations"]), pre["cov3D"], n(cam.world_view_transform),
                             n(cam.full_proj_transform), n(cam.camera_center), W, Hh, cam.tanfovx, cam.tanfovy, g2, gco,
                             gcol)
    gd = {k: H.dev(v) for k, v in g.items() if torch.is_tensor(v)}
    V, PM, cp = H.dev(cam.world_view_transform), H.dev(cam.full_proj_transform), H.dev(cam.camera_center)
    f = lambda *s: torch.full(s, 33.0, device=H.DEV)
    o = dict(dL_dmeans3D=f(P, 3), dL_dcov3D=f(P, 6), dL_dscales=f(P, 3), dL_drotations=f(P, 4), dL_dsh=f(P, 16, 3),
             dL_dopacity=f(P, 1))
    # keep every device tensor referenced until the call has run
    t_radii, t_cov, t_clamped = H.dev(pre["radii"]), H.dev(pre["cov3D"]), H.dev(pre["clamped"])
    t_g2, t_gco, t_gcol = H.dev(g2), H.dev(gco), H.dev(gcol)
    ddir = H.preprocess_fwd(g, cam, want_ddir=True)[0]["dcolor_ddir"] if saved else None
    H.gn.check(H.lib.gs_preprocess_backward(
        H.ptr(t_radii), H.ptr(t_cov), H.ptr(t_clamped), P, 3,
        16 if sh_mode else 0, W, Hh, H.ptr(gd["means3D"]), H.ptr(gd["scales"]), H.ptr(gd["rotations"]),
        H.ptr(gd["shs"]) if (sh_mode and not saved) else None, 1.0, H.ptr(V), H.ptr(PM), H.ptr(cp), cam.tanfovx,
        cam.tanfovy,
        H.ptr(t_g2), 2, H.ptr(t_gco), H.ptr(t_gcol), H.ptr(o["dL_dmeans3D"]), H.ptr(o["dL_dcov3D"]),
        H.ptr(o["dL_dscales"]), H.ptr(o["dL_drotations"]), H.ptr(o["dL_dsh"]) if sh_mode else None,
        H.ptr(o["dL_dopacity"]), 1, H.ptr(ddir) if saved else None, H.stream()), "gs_preprocess_backward")
    torch.cuda.synchronize()
    if saved:
        # against the same call with the coefficients: the same bits
        o2 = {k: torch.full_like(v, 33.0) for k, v in o.items()}
        H.gn.check(H.lib.gs_preprocess_backward(
            H.ptr(t_radii), H.ptr(t_cov), H.ptr(t_clamped), P, 3, 16, W, Hh, H.ptr(gd["means3D"]), H.ptr(gd["scales"]),
            H.ptr(gd["rotations"]), H.ptr(gd["shs"]), 1.0, H.ptr(V), H.ptr(PM), H.ptr(cp), cam.tanfovx, cam.tanfovy,
            H.ptr(t_g2), 2, H.ptr(t_gco), H.ptr(t_gcol), H.ptr(o2["dL_dmeans3D"]), H.ptr(o2["dL_dcov3D"]),
            H.ptr(o2["dL_dscales"]), H.ptr(o2["dL_drotations"]), H.ptr(o2["dL_dsh"]), H.ptr(o2["dL_dopacity"]), 1, None,
            H.stream()), "gs_preprocess_backward")
        torch.cuda.synchronize()
        for k in o:
            assert torch.equal(o[k], o2[k]), k
    # without the stored covariances (formed again from scales and rotations): the same bits
    o3 = {k: torch.full_like(v, 33.0) for k, v in o.items()}
    H.gn.check(H.lib.gs_preprocess_backward(
        H.ptr(t_radii), None, H.ptr(t_clamped), P, 3, 16 if sh_mode else 0, W, Hh, H.ptr(gd["means3D"]),
        H.ptr(gd["scales"]), H.ptr(gd["rotations"]), H.ptr(gd["shs"]) if (sh_mode and not saved) else None, 1.0,
        H.ptr(V), H.ptr(PM), H.ptr(cp), cam.tanfovx, cam.tanfovy, H.ptr(t_g2), 2, H.ptr(t_gco), H.ptr(t_gcol),
        H.ptr(o3["dL_dmeans3D"]), H.ptr(o3["dL_dcov3D"]), H.ptr(o3["dL_dscales"]), H.ptr(o3["dL_drotations"]),
        H.ptr(o3["dL_dsh"]) if sh_mode else None, H.ptr(o3["dL_dopacity"]), 1, H.ptr(ddir) if saved else None,
        H.stream()), "gs_preprocess_backward")
    torch.cuda.synchronize()
    for k in o:
        assert torch.equal(o[k], o3[k]), k
    keys = ["dL_dmeans3D", "dL_dcov3D", "dL_dscales", "dL_drotations", "dL_dopacity"] + (["dL_dsh"] if sh_mode else [])
    for k in keys:
        a, r = o[k].cpu().numpy(), ref[k]
        assert np.isfinite(a).all(), k
        assert H.rel_l2(a, r) <= GRAD_TOL, f"{k}: rel L2 {H.rel_l2(a, r)}"
        assert np.array_equal(a, r) or H.rel_l2(a, r) < 1e-6, f"{k} drifted from the op-for-op statement"


def _poison(g, seed=0):
    """Non-finite and absurd parameters in 2 % of the Gaussians (what a diverged optimisation hands the rasterizer)."""
    P = g["means3D"].shape[0]
    gen = torch.Generator().manual_seed(seed)
    idx = torch.randperm(P, generator=gen)[: P // 50].reshape(10, -1)
    nan, inf = float("nan"), float("inf")
    g["means3D"][idx[0], 0] = nan
    g["means3D"][idx[1], 2] = inf
    g["means3D"][idx[2]] = -inf
    g["scales"][idx[3], 1] = nan
    g["scales"][idx[4]] = inf
    g["scales"][idx[5]] = 1e20
    g["scales"][idx[6], 0] = -3.0
    g["rotations"][idx[7], 2] = nan
    g["rotations"][idx[8]] = 0.0
    g["opacities"][idx[9]] = nan
    return idx.reshape(-1)


@pytest.mark.parametrize("cfg,P", [(0, 40_000), (1, 100_000)])
def test_non_finite_parameters_are_contained(H, orc, cfg, P):
    """NaN, infinite and absurd means, scales, rotations and opacities: every kernel finishes, the integer outputs
    are the oracle's (a Gaussian whose radius or rectangle cannot be computed is culled, as by the saturating
    casts of cuda_rasterizer/auxiliary.h:66-76), and whatever the other Gaussians contribute stays finite."""
    import gs_scenes
    from diff_gaussian_rasterization import _C
    DEV = H.DEV
    g, cam = _scene(cfg, P)
    bad = _poison(g)
    got, gd = H.preprocess_fwd(g, cam)
    ref = H.oracle_preprocess(orc, g, cam)
    assert np.array_equal(got["radii"].cpu().numpy(), ref["radii"])
    assert np.array_equal(H.np_u32(got["tiles_touched"]), ref["tiles_touched"])
    radii = got["radii"]
    W, Hh = cam.image_width, cam.image_height
    gx, gy = H.grid(W, Hh)
    assert int(got["tiles_touched"].max()) <= gx * gy
    good = torch.ones(P, dtype=torch.bool)
    good[bad] = False
    good = good.to(DEV)
    for k in ("means2D", "depths", "conic_opacity", "rgb"):
        assert bool(torch.isfinite(got[k][good & (radii > 0)]).all()), k
    # lists and blending: same lists as the oracle builds from the same per-Gaussian outputs
    cl = torch.ones(gy, gx, dtype=torch.bool)
    n = lambda t: t.detach().cpu().numpy()
    want = orc.bin_and_sort(n(radii), n(got["means2D"]), n(got["depths"]), cl.numpy().reshape(-1), W, Hh)
    vm, cp = cam.world_view_transform.to(DEV), cam.camera_center.to(DEV)
    am = torch.zeros(P, 5, device=DEV)
    args = {"stats_collector": {}}
    out = _C.render_gaussians(torch.zeros(3, device=DEV), Hh, W, got["means2D"], got["depths"], radii,
                              got["conic_opacity"], got["rgb"], cl.to(DEV), vm, cp, cam.tanfovx, cam.tanfovy, am,
                              True, False, args)
    R, color, n_render, oam, geomB, binB, imgB = out[0], out[1], out[2], out[6], out[8], out[9], out[10]
    assert R == want["point_list"].shape[0]
    counts = want["ranges"].reshape(-1, 2).astype(np.int64)
    assert np.array_equal(n(n_render), (counts[:, 1] - counts[:, 0]).astype(np.int32))
    ug = gs_scenes.upstream_grads(cam)
    back = _C.render_gaussians_backward(torch.zeros(3, device=DEV), cam.tanfovx, cam.tanfovy, oam, am, R, geomB, binB,
                                        imgB, cl.to(DEV), ug["color"].to(DEV), ug["all_map"].to(DEV),
                                        ug["plane_depth"].to(DEV), got["means2D"], got["conic_opacity"], got["rgb"],
                                        True, False, args)
    for t in back:
        assert t.shape[0] == P
        assert float(t[radii == 0].abs().max()) == 0.0  # nothing reaches a culled Gaussian


@pytest.mark.parametrize("seed,W,Hh,geo", [(0, 100, 70, True), (1, 48, 48, False), (2, 161, 33, True)])
def test_blend_with_arbitrary_splats(H, orc, seed, W, Hh, geo):
    """The blend kernels on splats no preprocess would produce: indefinite and degenerate conics (power > 0 is a
    skip, forward.cu:375-376), opacities above 1 (alpha clamps at 0.99, :383), opaque stacks that end a pixel early,
    negative and large colours, image sizes with partial tiles.  Forward counters exact, images and gradients
    within tolerance."""
    gen = torch.Generator().manual_seed(200 + seed)
    P = 4000
    gx, gy = H.grid(W, Hh)
    means2D = (torch.rand(P, 2, generator=gen) * torch.tensor([W + 20.0, Hh + 20.0]) - 10.0).numpy()
    radii = torch.randint(1, 30, (P,), generator=gen, dtype=torch.int32).numpy()
    a = torch.rand(P, generator=gen) * 0.3 + 0.002
    c = torch.rand(P, generator=gen) * 0.3 + 0.002
    b = (torch.rand(P, generator=gen) * 2 - 1) * torch.sqrt(a * c) * 1.3  # |b| > sqrt(ac) for some: indefinite
    kind = torch.randint(0, 12, (P,), generator=gen)
    a[kind == 0] = 0.0
    c[kind == 1] = -0.05
    opac = torch.rand(P, generator=gen) * 1.2
    opac[kind == 2] = 5.0
    opac[kind == 3] = 0.0
    co = torch.stack([a, b, c, opac], 1).numpy()
    rgb = (torch.randn(P, 3, generator=gen) * 2).numpy()
    am = (torch.randn(P, 5, generator=gen)).numpy()
    depths = (torch.rand(P, generator=gen) * 50 + 0.3).numpy()
    cl = np.ones(gx * gy, bool)
    bins = orc.bin_and_sort(radii, means2D, depths, cl, W, Hh)
    bg = np.array([0.1, 0.7, 0.3], np.float32)
    tanx, tany = 0.8, 0.8 * Hh / W
    ref = orc.render_fwd(bins["ranges"], bins["point_list"], means2D, rgb, am, co, cl, bg, W, Hh, tanx, tany,
                         render_geo=geo)
    got = H.render_fwd(P, W, Hh, tanx, tany, H.as_u32(bins["ranges"]), H.as_u32(bins["point_list"]), H.dev(means2D),
                       H.dev(rgb), H.dev(am), H.dev(co), H.dev(cl), H.dev(bg), render_geo=geo)
    for k in ("n_contrib", "n_contrib2loss"):
        assert np.array_equal(H.np_u32(got[k]), ref[k]), k
    assert np.array_equal(got["out_observe"].cpu().numpy(), ref["out_observe"])
    assert (ref["final_T"] < 1e-3).any() and (ref["n_contrib"] < bins["ranges"].reshape(-1, 2)[:, 1].max()).any()
    assert np.abs(got["final_T"].cpu().numpy() - ref["final_T"]).max() <= IMG_TOL
    scale = max(1.0, float(np.abs(ref["color"]).max()))
    assert np.abs(got["color"].cpu().numpy() - ref["color"]).max() <= IMG_TOL * scale
    if geo:
        scale = max(1.0, float(np.abs(ref["out_all_map"]).max()))
        assert np.abs(got["out_all_map"].cpu().numpy() - ref["out_all_map"]).max() <= IMG_TOL * scale
    gen2 = torch.Generator().manual_seed(seed)
    gpix = torch.randn(3, Hh, W, generator=gen2).numpy()
    gmap = torch.randn(5, Hh, W, generator=gen2).numpy()
    gdep = np.zeros((1, Hh, W), np.float32)  # (plane depth divides by a blended normal: arbitrary here)
    rb = orc.render_bwd(bins["ranges"], bins["point_list"], means2D, co, rgb, am, ref["out_all_map"], ref["final_T"],
                        ref["n_contrib"], cl, bg, gpix, gmap, gdep, W, Hh, tanx, tany, render_geo=geo)
    gb = H.render_bwd(P, W, Hh, tanx, tany, H.dev(bg), H.as_u32(bins["ranges"]), H.as_u32(bins["point_list"]),
                      H.dev(means2D), H.dev(co), H.dev(rgb), H.dev(am), H.dev(ref["out_all_map"]),
                      H.dev(ref["final_T"]), H.as_u32(ref["n_contrib"]), H.dev(cl), H.dev(gpix), H.dev(gmap),
                      H.dev(gdep), H.as_u32(bins["emission_sorted"]), H.as_u32(bins["point_offsets"]), render_geo=geo)
    pairs = [("dL_dmeans2D", rb["dL_dmeans2D"][:, :2]), ("dL_dconic_opacity", rb["dL_dconic_opacity"]),
             ("dL_dcolors", rb["dL_dcolors"])] + ([("dL_dall_map", rb["dL_dall_map"])] if geo else [])
    for k, r in pairs:
        g_ = gb[k].cpu().numpy()
        assert np.isfinite(g_).all(), k
        assert H.rel_l2(g_, r) <= GRAD_TOL, f"{k}: rel L2 {H.rel_l2(g_, r)}"


@pytest.mark.parametrize("seed,reach", [(0, 300.0), (1, 3000.0), (2, 30000.0)])
def test_long_thin_splats_far_from_their_centre(H, orc, seed, reach):
    """Splats whose conic has one eigenvalue near the dilation limit (3.3) and one tiny, centred up to `reach`
    pixels outside the image along their long axis, so that a band a few pixels wide crosses the image.  There
    the three terms of the exponent (forward.cu:373) are many orders larger than their sum, and the per-pixel
    value is dominated by rounding: whatever it is, the per-block culling must never drop a splat that one of the
    block's pixels blends, so counters stay exact against the per-pixel oracle."""
    gen = torch.Generator().manual_seed(900 + seed)
    P, W, Hh = 400, 96, 64
    gx, gy = H.grid(W, Hh)
    through = torch.rand(P, 2, generator=gen, dtype=torch.float64) * torch.tensor([W - 1.0, Hh - 1.0])
    ang = torch.rand(P, generator=gen, dtype=torch.float64) * math.pi
    far = (torch.rand(P, generator=gen, dtype=torch.float64) * 2 - 1) * reach
    lam_big = torch.rand(P, generator=gen, dtype=torch.float64) * 2.8 + 0.5
    lam_small = 10.0 ** (-(torch.rand(P, generator=gen, dtype=torch.float64) * 4 + 4))   # 1e-4 .. 1e-8
    ux, uy = torch.cos(ang), torch.sin(ang)          # the long axis (small eigenvalue)
    means2D = torch.stack([through[:, 0] + far * ux, through[:, 1] + far * uy], 1).float().numpy()
    a = (lam_small * ux * ux + lam_big * uy * uy)
    b = ((lam_small - lam_big) * ux * uy)
    c = (lam_small * uy * uy + lam_big * ux * ux)
    opac = torch.rand(P, generator=gen) * 0.7 + 0.3
    co = torch.stack([a.float(), b.float(), c.float(), opac], 1).numpy()
    radii = np.full(P, 1 << 20, np.int32)            # every splat is listed in every tile
    rgb = torch.rand(P, 3, generator=gen).numpy()
    am = torch.randn(P, 5, generator=gen).numpy()
    depths = (torch.rand(P, generator=gen) * 50 + 0.3).numpy()
    cl = np.ones(gx * gy, bool)
    bins = orc.bin_and_sort(radii, means2D, depths, cl, W, Hh)
    bg = np.zeros(3, np.float32)
    tanx, tany = 0.8, 0.8 * Hh / W
    ref = orc.render_fwd(bins["ranges"], bins["point_list"], means2D, rgb, am, co, cl, bg, W, Hh, tanx, tany,
                         render_geo=True)
    got = H.render_fwd(P, W, Hh, tanx, tany, H.as_u32(bins["ranges"]), H.as_u32(bins["point_list"]), H.dev(means2D),
                       H.dev(rgb), H.dev(am), H.dev(co), H.dev(cl), H.dev(bg), render_geo=True)
    assert ref["n_contrib2loss"].sum() > 10 * W   # the bands do cross the image
    for k in ("n_contrib", "n_contrib2loss"):
        assert np.array_equal(H.np_u32(got[k]), ref[k]), k
    assert np.array_equal(got["out_observe"].cpu().numpy(), ref["out_observe"])
    assert np.array_equal(got["final_T"].cpu().numpy(), ref["final_T"])
    assert np.array_equal(got["color"].cpu().numpy(), ref["color"])


def test_needles_through_the_whole_forward_pass(H, orc):
    """Needle-shaped Gaussians (one axis 10^3 to 10^5 times the others, tens to hundreds of metres long) around
    and in front of the camera: after projection their conics have one eigenvalue at the dilation limit and one
    near zero, radii of tens of thousands of pixels and centres far outside the image.  Preprocess, lists and
    blend against the oracle: every integer exact, the images the same bits."""
    import gs_scenes
    P = 3000
    g, cam = _scene(0, P)
    gen = torch.Generator().manual_seed(77)
    W, Hh = cam.image_width, cam.image_height
    g = dict(g)
    length = 10.0 ** (torch.rand(P, generator=gen) * 1.5 + 0.7)          # 5 .. 160
    thin = 10.0 ** (-(torch.rand(P, 2, generator=gen) * 2 + 1))            # 1e-1 .. 1e-3
    g["scales"] = torch.cat([length[:, None], thin], 1)
    q = torch.randn(P, 4, generator=gen)
    g["rotations"] = q / q.norm(dim=1, keepdim=True)
    g["opacities"] = torch.rand(P, 1, generator=gen) * 0.6 + 0.4
    pre = H.oracle_preprocess(orc, g, cam)
    got_pre, _ = H.preprocess_fwd(g, cam)
    assert np.array_equal(got_pre["radii"].cpu().numpy(), pre["radii"])
    assert np.array_equal(H.np_u32(got_pre["depths"].view(torch.int32)), pre["depths"].view(np.uint32))
    for k in ("means2D", "conic_opacity", "rgb"):
        assert np.array_equal(got_pre[k].cpu().numpy(), pre[k], equal_nan=True), k
    assert (pre["radii"] > 5000).sum() > P // 10   # the needles are what they are meant to be
    gx, gy = H.grid(W, Hh)
    cl = np.ones(gx * gy, bool)
    b = orc.bin_and_sort(pre["radii"], pre["means2D"], pre["depths"], cl, W, Hh)
    am = gs_scenes.build_all_map(g["means3D"], g["scales"], g["rotations"], cam).numpy()
    bg = np.zeros(3, np.float32)
    ref = orc.render_fwd(b["ranges"], b["point_list"], pre["means2D"], pre["rgb"], am, pre["conic_opacity"], cl, bg, W,
                         Hh, cam.tanfovx, cam.tanfovy, render_geo=True)
    got = H.render_fwd(P, W, Hh, cam.tanfovx, cam.tanfovy, H.as_u32(b["ranges"]), H.as_u32(b["point_list"]),
                       H.dev(pre["means2D"]), H.dev(pre["rgb"]), H.dev(am), H.dev(pre["conic_opacity"]), H.dev(cl),
                       H.dev(bg), render_geo=True)
    assert ref["n_contrib2loss"].sum() > W * Hh
    for k in ("n_contrib", "n_contrib2loss"):
        assert np.array_equal(H.np_u32(got[k]), ref[k]), k
    assert np.array_equal(got["out_observe"].cpu().numpy(), ref["out_observe"])
    assert np.array_equal(got["final_T"].cpu().numpy(), ref["final_T"])
    assert np.array_equal(got["color"].cpu().numpy(), ref["color"])
    # ... and back: the same contributors, so the sums differ by their order only
    ug = gs_scenes.upstream_grads(cam)
    gpix, gmap = ug["color"].numpy(), ug["all_map"].numpy()
    gdep = np.zeros((1, Hh, W), np.float32)
    rb = orc.render_bwd(b["ranges"], b["point_list"], pre["means2D"], pre["conic_opacity"], pre["rgb"], am,
                        ref["out_all_map"], ref["final_T"], ref["n_contrib"], cl, bg, gpix, gmap, gdep, W, Hh,
                        cam.tanfovx, cam.tanfovy, render_geo=True)
    gb = H.render_bwd(P, W, Hh, cam.tanfovx, cam.tanfovy, H.dev(bg), H.as_u32(b["ranges"]), H.as_u32(b["point_list"]),
                      H.dev(pre["means2D"]), H.dev(pre["conic_opacity"]), H.dev(pre["rgb"]), H.dev(am),
                      H.dev(ref["out_all_map"]), H.dev(ref["final_T"]), H.as_u32(ref["n_contrib"]), H.dev(cl),
                      H.dev(gpix), H.dev(gmap), H.dev(gdep), H.as_u32(b["emission_sorted"]),
                      H.as_u32(b["point_offsets"]), render_geo=True)
    for k, r in (("dL_dmeans2D", rb["dL_dmeans2D"][:, :2]), ("dL_dconic_opacity", rb["dL_dconic_opacity"]),
                 ("dL_dcolors", rb["dL_dcolors"]), ("dL_dall_map", rb["dL_dall_map"])):
        a = gb[k].cpu().numpy()
        assert np.isfinite(a).all(), k
        assert H.rel_l2(a, r) <= GRAD_TOL, f"{k}: rel L2 {H.rel_l2(a, r)}"


@pytest.mark.parametrize("geo", [True, False])
def test_non_finite_colours_reach_only_the_pixels_that_blend_them(H, orc, geo):
    """A Gaussian whose colour or geometry channels are NaN or infinite (what a diverging training step hands the
    rasterizer) poisons exactly the pixels that blend it and the gradients that depend on those pixels, as in the
    reference (forward.cu:381-407, backward.cu:463-472) and the oracle; every other pixel and gradient keeps the
    bits / the value it has without it."""
    import gs_scenes
    g, cam, pre, cl, b, am = _render_inputs(H, orc, 0, 30_000, "all")
    W, Hh = cam.image_width, cam.image_height
    P = 30_000
    rgb, am = pre["rgb"].copy(), am.copy()
    vis = np.flatnonzero(pre["radii"] > 0)
    rng = np.random.default_rng(5)
    pick = rng.choice(vis, 40, replace=False)
    rgb[pick[:10], 0] = np.nan
    rgb[pick[10:20], 2] = np.inf
    am[pick[20:30], 1] = np.nan
    am[pick[30:40], 4] = -np.inf
    bg = np.array([0.1, 0.2, 0.3], np.float32)
    ref = orc.render_fwd(b["ranges"], b["point_list"], pre["means2D"], rgb, am, pre["conic_opacity"], cl, bg, W, Hh,
                         cam.tanfovx, cam.tanfovy, render_geo=geo)
    got = H.render_fwd(P, W, Hh, cam.tanfovx, cam.tanfovy, H.as_u32(b["ranges"]), H.as_u32(b["point_list"]),
                       H.dev(pre["means2D"]), H.dev(rgb), H.dev(am), H.dev(pre["conic_opacity"]), H.dev(cl),
                       H.dev(bg), render_geo=geo)
    for k in ("n_contrib", "n_contrib2loss"):
        assert np.array_equal(H.np_u32(got[k]), ref[k]), k
    assert np.array_equal(got["final_T"].cpu().numpy(), ref["final_T"])
    for k in (("color", "out_all_map") if geo else ("color",)):
        a, r = got[k].cpu().numpy(), ref[k]
        assert np.array_equal(np.isnan(a), np.isnan(r)), k
        assert np.array_equal(a[~np.isnan(r)], r[~np.isnan(r)]), k
        assert np.isnan(r).any() and np.isnan(r).mean() < 0.2, k  # poisoned pixels exist and stay few
    ug = gs_scenes.upstream_grads(cam)
    gpix, gmap = ug["color"].numpy(), ug["all_map"].numpy()
    gdep = np.zeros((1, Hh, W), np.float32)
    amp = np.where(np.isfinite(ref["out_all_map"]), ref["out_all_map"], 0.0).astype(np.float32)
    rb = orc.render_bwd(b["ranges"], b["point_list"], pre["means2D"], pre["conic_opacity"], rgb, am, amp,
                        ref["final_T"], ref["n_contrib"], cl, bg, gpix, gmap, gdep, W, Hh, cam.tanfovx, cam.tanfovy,
                        render_geo=geo)
    gb = H.render_bwd(P, W, Hh, cam.tanfovx, cam.tanfovy, H.dev(bg), H.as_u32(b["ranges"]), H.as_u32(b["point_list"]),
                      H.dev(pre["means2D"]), H.dev(pre["conic_opacity"]), H.dev(rgb), H.dev(am), H.dev(amp),
                      H.dev(ref["final_T"]), H.as_u32(ref["n_contrib"]), H.dev(cl), H.dev(gpix), H.dev(gmap),
                      H.dev(gdep), H.as_u32(b["emission_sorted"]), H.as_u32(b["point_offsets"]), render_geo=geo)
    pairs = [("dL_dmeans2D", rb["dL_dmeans2D"][:, :2]), ("dL_dconic_opacity", rb["dL_dconic_opacity"]),
             ("dL_dcolors", rb["dL_dcolors"])] + ([("dL_dall_map", rb["dL_dall_map"])] if geo else [])
    for k, r in pairs:
        a = gb[k].cpu().numpy()
        assert np.array_equal(np.isfinite(a), np.isfinite(r)), (k, int((np.isfinite(a) != np.isfinite(r)).sum()))
        ok = np.isfinite(r)
        # (the colour and channel gradients are weight x upstream gradient and stay finite throughout)
        assert ok.all() if k in ("dL_dcolors", "dL_dall_map") else ((~ok).any() and (~ok).mean() < 0.5), k
        assert H.rel_l2(a[ok], r[ok]) <= GRAD_TOL, k


@pytest.mark.parametrize("cfg,P,mask,geo", [(1, 150_000, "all", True), (1, 100_000, "rows", True),
                                            (3, 60_000, "checker", False)])
def test_backward_blend_gives_the_same_bits_with_the_forward_lists_and_with_its_own(H, orc, cfg, P, mask, geo):
    """The whole-view entry points hand the backward blend the row lists the forward blend built (16 bits per
    sorted instance in the binning buffer); the stage entry points have no such buffer and the backward blend tests
    every Gaussian against its blocks itself.  Same visits either way, so the five gradient tensors are the same
    bits."""
    import gs_scenes
    from diff_gaussian_rasterization import _C
    g, cam, pre, cl, b, am = _render_inputs(H, orc, cfg, P, mask)
    W, Hh = cam.image_width, cam.image_height
    gx, gy = H.grid(W, Hh)
    bg = np.array([0.2, 0.4, 0.6], np.float32)
    ug = gs_scenes.upstream_grads(cam)
    d = {k: H.dev(pre[k]) for k in ("means2D", "depths", "conic_opacity", "rgb")}
    radii = torch.from_numpy(pre["radii"].astype(np.int32)).to(H.DEV)
    t_am, t_cl, t_bg = H.dev(am), torch.from_numpy(cl.reshape(gy, gx)).to(H.DEV), H.dev(bg)
    gpix, gmap, gdep = (ug[k].to(H.DEV) for k in ("color", "all_map", "plane_depth"))
    vm, cp = cam.world_view_transform.to(H.DEV), cam.camera_center.to(H.DEV)

    args = {"stats_collector": {}}
    out, info = _C.render_gaussians_ex(t_bg, Hh, W, d["means2D"], d["depths"], radii, d["conic_opacity"], d["rgb"],
                                       t_cl, vm, cp, cam.tanfovx, cam.tanfovy, t_am, geo, False, args)
    whole = _C.render_gaussians_backward(t_bg, cam.tanfovx, cam.tanfovy, out[6], t_am, out[0], out[8], out[9],
                                         out[10], t_cl, gpix, gmap, gdep, d["means2D"], d["conic_opacity"], d["rgb"],
                                         geo, False, args, binning_capacity=info["binning_capacity"])

    f = H.render_fwd(P, W, Hh, cam.tanfovx, cam.tanfovy, H.as_u32(b["ranges"]), H.as_u32(b["point_list"]),
                     d["means2D"], d["rgb"], t_am, d["conic_opacity"], H.dev(cl), t_bg, render_geo=geo)
    stage = H.render_bwd(P, W, Hh, cam.tanfovx, cam.tanfovy, t_bg, H.as_u32(b["ranges"]), H.as_u32(b["point_list"]),
                         d["means2D"], d["conic_opacity"], d["rgb"], t_am, f["out_all_map"], f["final_T"],
                         f["n_contrib"], H.dev(cl), gpix, gmap, gdep, H.as_u32(b["emission_sorted"]),
                         H.as_u32(b["point_offsets"]), render_geo=geo)
    names = ["dL_dmeans2D", "dL_dmeans2D_abs", "dL_dconic_opacity", "dL_dcolors"] + (["dL_dall_map"] if geo else [])
    for k, a in zip(names, whole):
        assert torch.equal(a, stage[k]), k
    assert float(stage["dL_dcolors"].abs().max()) > 0.0
