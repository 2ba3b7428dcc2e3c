"""Writes tests/golden/tiny_scene.npz: inputs and expected outputs of one small
view (BASELINE config 0 distribution, 600 Gaussians, 96x64 image) computed by
the CPU oracle after it passed tests/test_oracle_pins.py.  The reference holds
no golden vectors for this path; this fixture freezes the pinned oracle so
that later edits to it (or a different compiler) are noticed, and gives the
GPU tests a second, file-based expectation.

Run from the repo root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "citygs-x_amd"))

import gs_scenes  # noqa: E402
from oracle import oracle as orc  # noqa: E402


def main():
    import torch
    P, W, H = 600, 96, 64
    g, _ = gs_scenes.make_scene(0, P=P, seed=7)
    g["scales"] = g["scales"] * 40.0  # larger splats so the small image has overlap and saturating pixels
    cam = gs_scenes.look_at_camera((0.0, 0.0, -30.0), (0, 0, 0), W, H, 60.0, up=(0.0, -1.0, 0.0))
    n = lambda t: t.numpy()
    pre = orc.preprocess_fwd(n(g["means3D"]), n(g["scales"]), n(g["rotations"]), n(g["opacities"]), n(g["shs"]),
                             n(cam.world_view_transform), n(cam.full_proj_transform), n(cam.camera_center), W, H,
                             cam.tanfovx, cam.tanfovy)
    gx, gy = orc.tile_grid(W, H)
    cl = np.ones(gx * gy, bool)
    b = orc.bin_and_sort(pre["radii"], pre["means2D"], pre["depths"], cl, W, H)
    am = gs_scenes.build_all_map(g["means3D"], g["scales"], g["rotations"], cam).numpy()
    bg = np.array([0.1, 0.2, 0.3], np.float32)
    f = orc.render_fwd(b["ranges"], b["point_list"], pre["means2D"], pre["rgb"], am, pre["conic_opacity"], cl, bg, W, H,
                       cam.tanfovx, cam.tanfovy)
    ug = gs_scenes.upstream_grads(cam, seed=7)
    rb = orc.render_bwd(b["ranges"], b["point_list"], pre["means2D"], pre["conic_opacity"], pre["rgb"], am,
                        f["out_all_map"], f["final_T"], f["n_contrib"], cl, bg, n(ug["color"]), n(ug["all_map"]),
                        n(ug["plane_depth"]), W, H, cam.tanfovx, cam.tanfovy)
    pb = orc.preprocess_bwd(n(g["means3D"]), pre["radii"], n(g["shs"]), pre["clamped"], n(g["scales"]),
                            n(g["rotations"]), pre["cov3D"], n(cam.world_view_transform), n(cam.full_proj_transform),
                            n(cam.camera_center), W, H, cam.tanfovx, cam.tanfovy, rb["dL_dmeans2D"],
                            rb["dL_dconic_opacity"], rb["dL_dcolors"])
    knn = orc.knn_dist2(n(g["means3D"]))
    out = dict(
        W=W, H=H, tanfovx=cam.tanfovx, tanfovy=cam.tanfovy, bg=bg,
        viewmatrix=n(cam.world_view_transform), projmatrix=n(cam.full_proj_transform), campos=n(cam.camera_center),
        means3D=n(g["means3D"]), scales=n(g["scales"]), rotations=n(g["rotations"]), opacities=n(g["opacities"]),
        shs=n(g["shs"]), all_map=am, g_color=n(ug["color"]), g_all_map=n(ug["all_map"]),
        g_plane_depth=n(ug["plane_depth"]),
        radii=pre["radii"], means2D=pre["means2D"], depths=pre["depths"], conic_opacity=pre["conic_opacity"],
        rgb=pre["rgb"], clamped=pre["clamped"], cov3D=pre["cov3D"], tiles_touched=pre["tiles_touched"],
        keys=b["keys"], point_list=b["point_list"], ranges=b["ranges"],
        color=f["color"], out_all_map=f["out_all_map"], out_plane_depth=f["out_plane_depth"], final_T=f["final_T"],
        n_contrib=f["n_contrib"], n_contrib2loss=f["n_contrib2loss"], out_observe=f["out_observe"],
        n_render=f["n_render"], n_consider=f["n_consider"], n_contrib_tile=f["n_contrib_tile"],
        dL_dmeans2D=rb["dL_dmeans2D"], dL_dmeans2D_abs=rb["dL_dmeans2D_abs"],
        dL_dconic_opacity=rb["dL_dconic_opacity"], dL_dcolors=rb["dL_dcolors"], dL_dall_map=rb["dL_dall_map"],
        dL_dmeans3D=pb["dL_dmeans3D"], dL_dscales=pb["dL_dscales"], dL_drotations=pb["dL_drotations"],
        dL_dsh=pb["dL_dsh"], knn_dist2=knn)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tiny_scene.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes; R =", b["num_rendered"], "mean n_contrib =",
          f["n_contrib"].mean(), "saturated px =", int((f["final_T"] < 0.01).sum()))


if __name__ == "__main__":
    main()
