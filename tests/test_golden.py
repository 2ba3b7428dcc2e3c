"""tests/golden/tiny_scene.npz (written by tests/golden/make_golden.py) against
the CPU oracle (CPU test) and against the HIP library (GPU test)."""
import os

import numpy as np
import pytest
import torch

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tiny_scene.npz")


@pytest.fixture(scope="module")
def gold():
    return dict(np.load(GOLD, allow_pickle=False))


def _rel(a, b):
    a, b = np.asarray(a, np.float64).ravel(), np.asarray(b, np.float64).ravel()
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


def test_oracle_reproduces_golden(orc, gold):
    g = gold
    W, H, tx, ty = int(g["W"]), int(g["H"]), float(g["tanfovx"]), float(g["tanfovy"])
    pre = orc.preprocess_fwd(g["means3D"], g["scales"], g["rotations"], g["opacities"], g["shs"], g["viewmatrix"],
                             g["projmatrix"], g["campos"], W, H, tx, ty)
    for k in ("radii", "means2D", "depths", "conic_opacity", "rgb", "clamped", "cov3D", "tiles_touched"):
        assert np.array_equal(pre[k], g[k]), k
    gx, gy = orc.tile_grid(W, H)
    cl = np.ones(gx * gy, bool)
    b = orc.bin_and_sort(pre["radii"], pre["means2D"], pre["depths"], cl, W, H)
    for k in ("keys", "point_list", "ranges"):
        assert np.array_equal(b[k], g[k]), k
    f = orc.render_fwd(b["ranges"], b["point_list"], pre["means2D"], pre["rgb"], g["all_map"], pre["conic_opacity"], cl,
                       g["bg"], W, H, tx, ty)
    for k in ("color", "out_all_map", "out_plane_depth", "final_T", "n_contrib", "n_contrib2loss", "out_observe",
              "n_render", "n_consider", "n_contrib_tile"):
        assert np.array_equal(f[k], g[k]), k
    rb = orc.render_bwd(b["ranges"], b["point_list"], pre["means2D"], pre["conic_opacity"], pre["rgb"], g["all_map"],
                        f["out_all_map"], f["final_T"], f["n_contrib"], cl, g["bg"], g["g_color"], g["g_all_map"],
                        g["g_plane_depth"], W, H, tx, ty)
    for k in ("dL_dmeans2D", "dL_dmeans2D_abs", "dL_dconic_opacity", "dL_dcolors", "dL_dall_map"):
        assert _rel(rb[k], g[k]) <= 1e-6, k  # double accumulation: thread order can move the last bit only
    assert np.array_equal(orc.knn_dist2(g["means3D"]), g["knn_dist2"])
    assert (g["final_T"] < 0.01).sum() > 0 and (g["n_contrib"] != g["n_contrib2loss"]).any()


@pytest.mark.gpu
def test_gpu_reproduces_golden(gold):
    from diff_gaussian_rasterization import GaussianRasterizationSettings, GaussianRasterizer
    from simple_knn._C import distCUDA2
    g = gold
    dev = "cuda:0"
    W, H = int(g["W"]), int(g["H"])
    t = lambda k: torch.from_numpy(g[k]).to(dev)
    rs = GaussianRasterizationSettings(H, W, float(g["tanfovx"]), float(g["tanfovy"]), t("bg"), 1.0, t("viewmatrix"),
                                       t("projmatrix"), 3, t("campos"), False, True, False)
    rast = GaussianRasterizer(rs)
    leaf = {k: t(k).requires_grad_(True) for k in ("means3D", "scales", "rotations", "opacities", "shs")}
    ca = {"avoid_pixel_all2all": False, "stats_collector": {}}
    m2, rgb, co, radii, depths = rast.preprocess_gaussians(leaf["means3D"], leaf["scales"], leaf["rotations"],
                                                           leaf["shs"], leaf["opacities"], ca)
    n = lambda x: x.detach().cpu().numpy()
    assert np.array_equal(n(radii), g["radii"])
    assert np.array_equal(n(depths).view(np.uint32), g["depths"].view(np.uint32))
    for k, v in (("means2D", m2), ("conic_opacity", co), ("rgb", rgb)):
        assert np.abs(n(v) - g[k]).max() <= 1e-6 * max(1.0, np.abs(g[k]).max()), k
    gx, gy = (W + 15) // 16, (H + 15) // 16
    cl = torch.ones(gy, gx, dtype=torch.bool, device=dev)
    m2abs = torch.zeros(len(g["radii"]), 3, device=dev, requires_grad=True)
    color, n_render, n_consider, n_contrib, observe, oam, opd = rast.render_gaussians(m2, m2abs, co, rgb, t("all_map"),
                                                                                     depths, radii, cl, cl, ca)
    assert np.array_equal(n(n_render), g["n_render"]) and np.array_equal(n(n_consider), g["n_consider"])
    assert np.array_equal(n(n_contrib), g["n_contrib_tile"]) and np.array_equal(n(observe), g["out_observe"])
    assert np.abs(n(color) - g["color"]).max() <= 1e-4
    assert np.abs(n(oam) - g["out_all_map"]).max() <= 1e-4
    assert np.abs(n(opd) - g["out_plane_depth"]).max() <= 1e-4 * max(1.0, np.abs(g["out_plane_depth"]).max())
    torch.autograd.backward([color, oam, opd], [t("g_color"), t("g_all_map"), t("g_plane_depth")])
    assert _rel(n(m2abs.grad), g["dL_dmeans2D_abs"]) <= 1e-3
    for k, r in (("means3D", "dL_dmeans3D"), ("scales", "dL_dscales"), ("rotations", "dL_drotations"),
                 ("shs", "dL_dsh")):
        assert _rel(n(leaf[k].grad), g[r]) <= 1e-3, k
    assert _rel(n(leaf["opacities"].grad)[:, 0], g["dL_dconic_opacity"][:, 3]) <= 1e-3
    assert np.array_equal(distCUDA2(t("means3D")).cpu().numpy(), g["knn_dist2"])
