"""Randomised end-to-end parity: the whole pipeline (preprocess, per-tile lists, blend forward and backward,
preprocess backward) against the CPU oracle on random scenes, cameras, image sizes with partial tiles, tile masks,
geometry on/off and list routes.  Seeded: the same 40 cases every run."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
ROUTES = [(-1, -1), (0, 0), (40, 0), (7, 7), (300, 500)]


@pytest.fixture(scope="module")
def H():
    import gpu_harness
    return gpu_harness


@pytest.mark.parametrize("block", range(4))
def test_random_views_match_oracle(orc, H, block):
    import gs_scenes
    import gsrast_native as gn
    from diff_gaussian_rasterization import _C
    rng = np.random.default_rng(1000 + block)
    n = lambda t: t.detach().cpu().numpy()
    rendered = 0
    if True:
        for case in range(10):
            seed = int(rng.integers(1 << 30))
            cfg = int(rng.choice([0, 1, 3]))
            P = int(rng.choice([500, 3000, 20000, 60000]))
            W = int(rng.choice([64, 100, 333, 640, 800, 1152]))
            Hh = int(rng.choice([48, 70, 217, 480, 600]))
            g, _ = gs_scenes.make_scene(cfg, seed=seed, P=P, n_views=1)
            ext = {0: 10.0, 1: 100.0, 3: 300.0}[cfg]
            eye = (rng.uniform(-ext, ext), rng.uniform(-ext, ext), rng.uniform(1.0, ext))
            tgt = (rng.uniform(-ext / 2, ext / 2), rng.uniform(-ext / 2, ext / 2), rng.uniform(0, 5))
            cam = gs_scenes.look_at_camera(eye, tgt, W, Hh, float(rng.uniform(30, 100)))
            g["scales"] = g["scales"] + float(rng.uniform(-0.5, 1.0))
            gx, gy = H.grid(W, Hh)
            mk = rng.choice(["all", "rand", "rows"])
            cl = torch.ones(gy, gx, dtype=torch.bool)
            if mk == "rand":
                cl = torch.from_numpy(rng.random((gy, gx)) < 0.6)
            if mk == "rows":
                cl[: gy // 2] = False
            geo = bool(rng.integers(2))
            route = ROUTES[int(rng.integers(len(ROUTES)))]
            tag = f"block {block} case {case}: seed {seed} cfg {cfg} P {P} {W}x{Hh} mask {mk} geo {geo} route {route}"

            o, gd = H.preprocess_fwd(g, cam)
            ref = H.oracle_preprocess(orc, g, cam)
            assert np.array_equal(n(o["radii"]), ref["radii"]), tag
            assert np.array_equal(H.np_u32(o["tiles_touched"]), ref["tiles_touched"]), tag
            for k in ("means2D", "cov3D", "conic_opacity", "rgb"):
                assert np.array_equal(n(o[k]), ref[k]), (tag, k)
            clf = cl.numpy().reshape(-1)
            want = orc.bin_and_sort(ref["radii"], ref["means2D"], ref["depths"], clf, W, Hh)
            am = gs_scenes.build_all_map(gd["means3D"], gd["scales"], gd["rotations"], cam)
            bg = torch.tensor(rng.random(3), dtype=torch.float32, device=DEV)
            args = {"stats_collector": {}, "tile_sort_limits": route}
            vm, pm, cp = cam.world_view_transform.to(DEV), cam.full_proj_transform.to(DEV), cam.camera_center.to(DEV)
            # what the caller says it expects of the view: nothing, enough, too little, or exactly right (the list
            # kernels and the blend are then launched ahead of the instance count, and redone if the view does not fit)
            R_want = int(want["point_list"].shape[0])
            counts = want["ranges"].reshape(-1, 2).astype(np.int64)
            longest_want = int((counts[:, 1] - counts[:, 0]).max())
            expect = str(rng.choice(["none", "enough", "too few", "exact", "list too long"]))
            exp_n, exp_l = {"none": (0, 0), "enough": (R_want + int(rng.integers(1, 5000)), 0),
                            "too few": (max(1, R_want // 2), 0), "exact": (max(1, R_want), longest_want),
                            "list too long": (R_want + 7, max(1, longest_want // 2))}[expect]
            tag += f" expect {expect}"
            out, info = _C.render_gaussians_ex(bg, Hh, W, o["means2D"], o["depths"], o["radii"], o["conic_opacity"],
                                               o["rgb"], cl.to(DEV), vm, cp, cam.tanfovx, cam.tanfovy, am, geo, False,
                                               args, expected_instances=exp_n, expected_longest_list=exp_l)
            R, color, n_render, n_consider, n_contrib, obs, oam, opd, geomB, binB, imgB = out
            assert R == R_want, tag
            assert info["binning_capacity"] == (exp_n if info["launched_ahead"] else R), tag
            if exp_n == 0 or exp_n < R_want or 0 < exp_l < longest_want:
                assert not info["launched_ahead"], tag
            rendered += R > 0
            f = orc.render_fwd(want["ranges"], want["point_list"], ref["means2D"], ref["rgb"], n(am),
                               ref["conic_opacity"], clf, n(bg), W, Hh, cam.tanfovx, cam.tanfovy, render_geo=geo)
            px = np.repeat(np.repeat(cl.numpy(), 16, 0), 16, 1)[:Hh, :W]
            assert np.array_equal(n(obs), f["out_observe"]), tag
            assert np.array_equal(n(n_render), f["n_render"]), tag
            assert np.array_equal(n(n_consider), f["n_consider"]), tag
            assert np.array_equal(n(n_contrib), f["n_contrib_tile"]), tag
            # images: the oracle's bits where computed, zero elsewhere
            assert np.array_equal(n(color), f["color"]), tag
            if geo:
                assert np.array_equal(n(oam), f["out_all_map"]), tag
                a, r = n(opd), f["out_plane_depth"]
                assert np.array_equal(np.isnan(a), np.isnan(r)), tag
                assert np.array_equal(a[~np.isnan(r)], r[~np.isnan(r)]), tag
            else:
                assert float(oam.abs().max()) == 0.0 and float(opd.abs().max()) == 0.0, tag
            ug = gs_scenes.upstream_grads(cam)
            # The plane-depth gradient divides by tmp = (blended normal . ray) twice; where that is almost zero the
            # gradient is astronomically large and says nothing about parity, so the upstream gradient is kept only
            # where the oracle's own tmp is at least 1e-3 in size.
            fx_, fy_ = W / (2.0 * cam.tanfovx), Hh / (2.0 * cam.tanfovy)
            rayx = (np.arange(W, dtype=np.float64)[None, :] - W * 0.5) / fx_
            rayy = (np.arange(Hh, dtype=np.float64)[:, None] - Hh * 0.5) / fy_
            om = f["out_all_map"].astype(np.float64)
            tmp = om[0] * rayx + om[1] * rayy + om[2]
            gdep = ug["plane_depth"] * torch.from_numpy((np.abs(tmp) >= 1e-3)[None].astype(np.float32))
            if not geo:
                gdep = torch.zeros_like(gdep)
            back = _C.render_gaussians_backward(bg, cam.tanfovx, cam.tanfovy, oam, am, R, geomB, binB, imgB,
                                                cl.to(DEV), ug["color"].to(DEV), ug["all_map"].to(DEV),
                                                gdep.to(DEV), o["means2D"], o["conic_opacity"], o["rgb"], geo, False,
                                                args, binning_capacity=info["binning_capacity"])
            rb = orc.render_bwd(want["ranges"], want["point_list"], ref["means2D"], ref["conic_opacity"], ref["rgb"],
                                n(am), f["out_all_map"], f["final_T"], f["n_contrib"], clf, n(bg), n(ug["color"]),
                                n(ug["all_map"]), n(gdep), W, Hh, cam.tanfovx, cam.tanfovy, render_geo=geo)
            for k, got, w in (("means2D", back[0][:, :2], rb["dL_dmeans2D"][:, :2]),
                              ("means2D_abs", back[1], rb["dL_dmeans2D_abs"]),
                              ("conic_opacity", back[2], rb["dL_dconic_opacity"]), ("colors", back[3], rb["dL_dcolors"]),
                              ("all_map", back[4], rb["dL_dall_map"])):
                assert np.isfinite(n(got)).all(), (tag, k)
                if np.linalg.norm(w) > 0:
                    assert H.rel_l2(n(got), w) <= 1e-3, (tag, k)
                else:
                    assert float(got.abs().max()) == 0.0, (tag, k)
            pb = _C.preprocess_gaussians_backward(o["radii"], o["cov3D"], o["clamped"].bool(), gd["means3D"],
                                                  gd["scales"], gd["rotations"], gd["shs"], 1.0, vm, pm, cam.tanfovx,
                                                  cam.tanfovy, Hh, W, 3, cp, back[0], back[2], back[3], R, False, args)
            ob = orc.preprocess_bwd(n(gd["means3D"]), ref["radii"], n(gd["shs"]), ref["clamped"], n(gd["scales"]),
                                    n(gd["rotations"]), ref["cov3D"], n(vm), n(pm), n(cp), W, Hh, cam.tanfovx,
                                    cam.tanfovy, n(back[0]), n(back[2]), n(back[3]), sh_degree=3)
            for k, got in zip(("dL_dmeans3D", "dL_dscales", "dL_drotations", "dL_dsh"), pb[:4]):
                if np.linalg.norm(ob[k]) > 0:
                    assert H.rel_l2(n(got).reshape(ob[k].shape), ob[k]) <= 1e-3, (tag, k)
    assert rendered >= 7  # the random cameras look at the scene in nearly every case
