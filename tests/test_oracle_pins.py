"""Pins for the CPU oracle (oracle/gs_oracle.cpp): closed forms, library
routines, brute force on tiny inputs and an independent torch restatement with
autograd.  The reference ships no tests or golden vectors for this path, so
these are what fixes the oracle's meaning.  CPU only."""
import math

import numpy as np
import pytest
import torch

import gs_scenes
from oracle import torch_ref as tr


def _cam(W=640, H=480, fov=60.0, eye=(0.0, 0.0, -30.0), tgt=(0, 0, 0), up=(0.0, -1.0, 0.0)):
    return gs_scenes.look_at_camera(eye, tgt, W, H, fov, up=up)


def _rel(a, b):
    a, b = np.asarray(a, np.float64).ravel(), np.asarray(b, np.float64).ravel()
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


def _pre(orc, g, cam, **kw):
    n = lambda t: t.numpy()
    return orc.preprocess_fwd(n(g["means3D"]), n(g["scales"]), n(g["rotations"]), n(g["opacities"]),
                              kw.pop("shs", n(g["shs"])), n(cam.world_view_transform), n(cam.full_proj_transform),
                              n(cam.camera_center), cam.image_width, cam.image_height, cam.tanfovx, cam.tanfovy, **kw)


# ------------------------------------------------------------------ scalars --

def test_expf_against_libm(orc):
    x = np.concatenate([np.linspace(-87, 0, 200001), np.linspace(0, 5, 1001), [-5.541264, -1e-8, 0.0]]).astype(np.float32)
    y = orc.expf(x)
    ref = np.exp(x.astype(np.float64))
    ulp = np.spacing(ref.astype(np.float32)).astype(np.float64)
    assert np.max(np.abs(y.astype(np.float64) - ref) / ulp) <= 1.5
    assert orc.expf(np.array([0.0], np.float32))[0] == 1.0
    assert orc.expf(np.array([-87.5, -1000.0], np.float32)).tolist() == [0.0, 0.0]
    xs = np.sort(x[x <= 0])
    assert (np.diff(orc.expf(xs)) >= 0).all()  # monotone: threshold tests cannot flip back and forth


def test_higher_msb(orc):
    for n in [1, 2, 3, 4, 255, 256, 1200, 3888, 4095, 4096, 8160, 65535, 65536, 1 << 20]:
        assert orc.higher_msb(n) == n.bit_length(), n
    assert orc.higher_msb(40 * 30) == 11 and orc.higher_msb(72 * 54) == 12 and orc.higher_msb(120 * 68) == 13


# --------------------------------------------------------------- preprocess --

def test_preprocess_closed_form_on_axis(orc):
    """Identity rotation, isotropic scale s, on the optical axis at depth z:
    cov2D = diag((f s / z)^2 + 0.3), radius = ceil(3 sqrt(.)), pixel = ((0+1) S - 1) / 2."""
    cam = _cam()
    W, H = 640, 480
    f = W / (2 * cam.tanfovx)
    for s, z in [(0.05, 30.0), (0.5, 10.0), (1.0, 55.0)]:
        g = dict(means3D=torch.tensor([[0.0, 0.0, z - 30.0]]), scales=torch.full((1, 3), s),
                 rotations=torch.tensor([[1.0, 0, 0, 0]]), opacities=torch.tensor([[0.7]]), shs=torch.zeros(1, 16, 3))
        o = _pre(orc, g, cam)
        var = (f * s / z) ** 2 + 0.3
        assert o["radii"][0] == math.ceil(3 * math.sqrt(var))
        np.testing.assert_allclose(o["means2D"][0], [(W - 1) / 2, (H - 1) / 2], rtol=0, atol=1e-3)
        np.testing.assert_allclose(o["conic_opacity"][0], [1 / var, 0, 1 / var, 0.7], rtol=2e-5, atol=1e-7)
        np.testing.assert_allclose(o["depths"][0], z, rtol=1e-6)
        np.testing.assert_allclose(o["cov3D"][0], [s * s, 0, 0, s * s, 0, s * s], rtol=1e-6, atol=1e-12)
        np.testing.assert_allclose(o["rgb"][0], [0.5, 0.5, 0.5])  # zero SH -> 0.5
        assert o["tiles_touched"][0] >= 1


@pytest.mark.parametrize("cfg", [0, 1])
def test_preprocess_matches_matrix_form(orc, cfg):
    g, cams = gs_scenes.make_scene(cfg, P=20_000)
    cam = cams[0]
    o = _pre(orc, g, cam)
    d = lambda t: t.double()
    r = tr.preprocess(d(g["means3D"]), d(g["scales"]), d(g["rotations"]), d(g["opacities"]),
                      d(cam.world_view_transform), d(cam.full_proj_transform), cam.image_width, cam.image_height,
                      cam.tanfovx, cam.tanfovy, shs=d(g["shs"]), campos=d(cam.camera_center))
    vis = o["radii"] > 0
    assert vis.sum() > 1000
    # invariant: dropped <=> behind the camera or empty tile rectangle (det == 0 never happens with the 0.3 filter)
    assert (r["in_front"].numpy()[vis]).all()
    for k, tol in (("means2D", 2e-6), ("depths", 1e-6), ("conic_opacity", 2e-5), ("rgb", 1e-5)):
        assert _rel(o[k][vis], r[k].numpy()[vis]) <= tol, k
    infront = r["in_front"].numpy()
    assert _rel(o["cov3D"][infront], np.stack([r["Sigma"][:, i, j].numpy() for i, j in
                                                ((0, 0), (0, 1), (0, 2), (1, 1), (1, 2), (2, 2))], 1)[infront]) <= 1e-6
    assert (o["cov3D"][~infront] == 0).all()
    rf = np.ceil(r["radius_f"].numpy())
    assert (np.abs(o["radii"][vis] - rf[vis]) <= 1).all() and (o["radii"][vis] == rf[vis]).mean() > 0.999
    assert np.array_equal(o["clamped"][vis].astype(bool), r["clamped"].numpy()[vis]) or \
        (o["clamped"][vis].astype(bool) != r["clamped"].numpy()[vis]).mean() < 1e-4
    # conic is the inverse of the filtered 2D covariance
    a, b, c = (r["cov2D"][:, i].numpy()[vis] for i in range(3))
    co = o["conic_opacity"][vis]
    np.testing.assert_allclose(co[:, 0] * a + co[:, 1] * b, 1.0, atol=1e-4)
    np.testing.assert_allclose(co[:, 0] * b + co[:, 1] * c, 0.0, atol=1e-4)
    # visibility prefilter and frustum mark agree with preprocess
    n = lambda t: t.numpy()
    vf = orc.visible_filter(n(g["means3D"]), n(g["scales"]), n(g["rotations"]), None, n(cam.world_view_transform),
                            n(cam.full_proj_transform), cam.image_width, cam.image_height, cam.tanfovx, cam.tanfovy)
    assert np.array_equal(vf, o["radii"])
    vf2 = orc.visible_filter(n(g["means3D"]), None, None, o["cov3D"], n(cam.world_view_transform),
                             n(cam.full_proj_transform), cam.image_width, cam.image_height, cam.tanfovx, cam.tanfovy)
    assert np.array_equal(vf2[infront], o["radii"][infront])
    mv = orc.mark_visible(n(g["means3D"]), n(cam.world_view_transform), n(cam.full_proj_transform))
    assert np.array_equal(mv, infront)


def test_reference_compatible_mode_leaves_colour_zero(orc):
    g, cams = gs_scenes.make_scene(0, P=500)
    o = _pre(orc, g, cams[0], shs=None)
    assert (o["rgb"] == 0).all() and (o["clamped"] == 0).all() and (o["radii"] > 0).any()


def test_sh_degree0_and_rotation_invariance(orc):
    g, cams = gs_scenes.make_scene(0, P=200)
    cam = cams[0]
    sh = torch.zeros(200, 16, 3)
    sh[:, 0] = torch.randn(200, 3, generator=torch.Generator().manual_seed(1))
    o = _pre(orc, g, cam, shs=sh.numpy(), sh_degree=0)
    vis = o["radii"] > 0
    np.testing.assert_allclose(o["rgb"][vis], np.maximum(0, 0.5 + tr.C0 * sh[:, 0].numpy()[vis]), atol=1e-6)
    # band-1 energy: sum_k B_k(d)^2 = C1^2 for every unit direction
    dirs = torch.nn.functional.normalize(torch.randn(50, 3, dtype=torch.float64), dim=-1)
    B = tr.sh_basis(dirs, 3)
    np.testing.assert_allclose((B[:, 1:4] ** 2).sum(-1).numpy(), tr.C1 ** 2, rtol=1e-12)
    np.testing.assert_allclose((B[:, 4:9] ** 2).sum(-1).numpy(), 5 / (4 * math.pi), rtol=1e-6)
    np.testing.assert_allclose((B[:, 9:16] ** 2).sum(-1).numpy(), 7 / (4 * math.pi), rtol=1e-6)


@pytest.mark.parametrize("cfg,deg", [(0, 3), (1, 3), (1, 1)])
def test_preprocess_backward_matches_autograd(orc, cfg, deg):
    P = 3000
    g, cams = gs_scenes.make_scene(cfg, P=P)
    cam = cams[0]
    W, H = cam.image_width, cam.image_height
    o = _pre(orc, g, cam, sh_degree=deg)
    vis = torch.from_numpy(o["radii"] > 0)
    gen = torch.Generator().manual_seed(11)
    g2 = torch.randn(P, 2, generator=gen, dtype=torch.float64)
    gco = torch.randn(P, 4, generator=gen, dtype=torch.float64)
    gcol = torch.randn(P, 3, generator=gen, dtype=torch.float64)
    leaves = {k: g[k].double().requires_grad_(True) for k in ("means3D", "scales", "rotations", "shs", "opacities")}
    r = tr.preprocess(leaves["means3D"], leaves["scales"], leaves["rotations"], leaves["opacities"],
                      cam.world_view_transform.double(), cam.full_proj_transform.double(), W, H, cam.tanfovx,
                      cam.tanfovy, shs=leaves["shs"], campos=cam.camera_center.double(), degree=deg)
    m = vis[:, None].double()
    # Convention between the two ops: the off-diagonal conic gradient that render backward emits is HALF the
    # derivative with respect to the conic's b entry (backward.cu:557 has the -0.5 factor on a term that enters the
    # exponent once), and preprocess backward doubles it back (backward.cu:135-137).  So a unit of gco[:,1] is
    # worth two units of true gradient.
    conv = torch.tensor([1.0, 2.0, 1.0, 1.0], dtype=torch.float64)
    loss = (r["ndc"][:, :2] * g2 * m).sum() + (r["conic_opacity"] * gco * conv * m).sum() + (r["rgb"] * gcol * m).sum()
    loss.backward()
    n = lambda t: t.numpy()
    b = orc.preprocess_bwd(n(g["means3D"]), o["radii"], n(g["shs"]), o["clamped"], n(g["scales"]), n(g["rotations"]),
                           o["cov3D"], n(cam.world_view_transform), n(cam.full_proj_transform), n(cam.camera_center), W,
                           H, cam.tanfovx, cam.tanfovy, g2.numpy(), gco.numpy(), gcol.numpy(), sh_degree=deg)
    assert _rel(b["dL_dmeans3D"], leaves["means3D"].grad.numpy()) <= 2e-4
    assert _rel(b["dL_dscales"], leaves["scales"].grad.numpy()) <= 2e-4
    assert _rel(b["dL_drotations"], leaves["rotations"].grad.numpy()) <= 2e-4
    assert _rel(b["dL_dsh"], leaves["shs"].grad.numpy()) <= 1e-5
    # opacity is a pass-through of the packed gradient (rasterize_points.cu:191-194): not masked by visibility
    np.testing.assert_array_equal(b["dL_dopacity"][:, 0], gco.numpy()[:, 3].astype(np.float32))
    assert (b["dL_dmeans3D"][~vis.numpy()] == 0).all() and (b["dL_dsh"][~vis.numpy()] == 0).all()


def test_cov3d_gradient_convention_and_finite_differences(orc):
    """dL/dcov3D doubles the off-diagonal entries (backward.cu:146-152); checked by central differences in
    float64 on the torch restatement, which the oracle must match."""
    g, cams = gs_scenes.make_scene(0, P=16)
    cam = cams[0]
    W, H = cam.image_width, cam.image_height
    o = _pre(orc, g, cam)
    gco = np.zeros((16, 4))
    gco[:, :3] = np.random.default_rng(0).normal(size=(16, 3))
    n = lambda t: t.numpy()
    b = orc.preprocess_bwd(n(g["means3D"]), o["radii"], n(g["shs"]), o["clamped"], n(g["scales"]), n(g["rotations"]),
                           o["cov3D"], n(cam.world_view_transform), n(cam.full_proj_transform), n(cam.camera_center), W,
                           H, cam.tanfovx, cam.tanfovy, np.zeros((16, 2)), gco, np.zeros((16, 3)))

    def f(sc):
        r = tr.preprocess(g["means3D"].double(), sc, g["rotations"].double(), g["opacities"].double(),
                          cam.world_view_transform.double(), cam.full_proj_transform.double(), W, H, cam.tanfovx,
                          cam.tanfovy)
        return float((r["conic_opacity"][:, :3] * torch.from_numpy(gco[:, :3]) * torch.tensor([1.0, 2.0, 1.0])).sum())
    sc = g["scales"].double()
    fd = np.zeros((16, 3))
    for i in range(16):
        for k in range(3):
            h = 1e-6 * float(sc[i, k])
            sp, sm = sc.clone(), sc.clone()
            sp[i, k] += h
            sm[i, k] -= h
            fd[i, k] = (f(sp) - f(sm)) / (2 * h)
    vis = o["radii"] > 0
    assert vis.all()
    assert _rel(b["dL_dscales"], fd) <= 1e-3


# ------------------------------------------------------------------ binning --

def test_binning_against_brute_force(orc):
    g, cams = gs_scenes.make_scene(0, P=4000)
    cam = cams[0]
    W, H = cam.image_width, cam.image_height
    o = _pre(orc, g, cam)
    gx, gy = orc.tile_grid(W, H)
    rng = np.random.default_rng(3)
    for cl in (np.ones(gx * gy, bool), rng.random(gx * gy) < 0.6):
        b = orc.bin_and_sort(o["radii"], o["means2D"], o["depths"], cl, W, H)
        # brute force: a tile is touched iff it intersects the pixel square [c - r, c + r] under the reference's
        # truncating rule, restated with integer tile bounds
        cnt = np.zeros(len(o["radii"]), np.uint32)
        keys, vals = [], []
        for i in np.nonzero(o["radii"] > 0)[0]:
            px, py = np.float32(o["means2D"][i, 0]), np.float32(o["means2D"][i, 1])
            r = np.float32(o["radii"][i])
            x0 = min(gx, max(0, int(np.float32(px - r) / np.float32(16))))
            y0 = min(gy, max(0, int(np.float32(py - r) / np.float32(16))))
            x1 = min(gx, max(0, int(np.float32(np.float32(np.float32(px + r) + np.float32(16)) - np.float32(1)) / np.float32(16))))
            y1 = min(gy, max(0, int(np.float32(np.float32(np.float32(py + r) + np.float32(16)) - np.float32(1)) / np.float32(16))))
            for y in range(y0, y1):
                for x in range(x0, x1):
                    if cl[y * gx + x]:
                        cnt[i] += 1
                        keys.append((np.uint64(y * gx + x) << np.uint64(32)) | np.uint64(o["depths"][i:i + 1].view(np.uint32)[0]))
                        vals.append(i)
        assert np.array_equal(b["tiles_touched"], cnt)
        assert np.array_equal(b["point_offsets"], np.cumsum(cnt, dtype=np.uint64).astype(np.uint32))
        keys, vals = np.array(keys, np.uint64), np.array(vals, np.uint32)
        assert np.array_equal(b["keys_unsorted"], keys) and np.array_equal(b["vals_unsorted"], vals)
        order = np.argsort(keys, kind="stable")
        assert np.array_equal(b["keys"], keys[order]) and np.array_equal(b["point_list"], vals[order])
        tiles = (b["keys"] >> np.uint64(32)).astype(np.int64)
        lo = np.searchsorted(tiles, np.arange(gx * gy), side="left")
        hi = np.searchsorted(tiles, np.arange(gx * gy), side="right")
        empty = lo == hi
        assert np.array_equal(b["ranges"][~empty, 0], lo[~empty]) and np.array_equal(b["ranges"][~empty, 1], hi[~empty])
        assert (b["ranges"][empty] == 0).all()
        if cl.all():
            assert np.array_equal(b["tiles_touched"], o["tiles_touched"])  # preprocess's rectangle area


def test_sort_is_stable_and_respects_bit_range(orc):
    rng = np.random.default_rng(5)
    keys = (rng.integers(0, 16, 5000, dtype=np.uint64) << np.uint64(32)) | rng.integers(0, 4, 5000, dtype=np.uint64)
    junk = rng.integers(0, 2, 5000, dtype=np.uint64) << np.uint64(50)
    vals = np.arange(5000, dtype=np.uint32)
    ko, vo = orc.sort_pairs(keys | junk, vals, 36)
    order = np.argsort(keys, kind="stable")
    assert np.array_equal(vo, vals[order]) and np.array_equal(ko, (keys | junk)[order])
    k32 = rng.integers(0, 100, 3000, dtype=np.uint32)
    ko, vo = orc.sort_pairs_u32(k32, np.arange(3000, dtype=np.uint32))
    assert np.array_equal(vo, np.argsort(k32, kind="stable").astype(np.uint32))


def test_empty_binning(orc):
    r = orc.tile_ranges(np.zeros(0, np.uint64), 12)
    assert r.shape == (12, 2) and (r == 0).all()
    b = orc.bin_and_sort(np.zeros(5, np.int32), np.zeros((5, 2), np.float32), np.zeros(5, np.float32), np.ones(1200, bool),
                         640, 480)
    assert b["num_rendered"] == 0 and (b["ranges"] == 0).all()


# ------------------------------------------------------------------- render --

def _one_gaussian(orc, mean, conic, opacity, rgb, amap, bg, W=48, H=32, geo=True):
    cam = _cam(W, H)
    gx, gy = orc.tile_grid(W, H)
    means2D = np.array([mean], np.float32)
    co = np.array([[conic[0], conic[1], conic[2], opacity]], np.float32)
    radii = np.array([200], np.int32)
    b = orc.bin_and_sort(radii, means2D, np.array([5.0], np.float32), np.ones(gx * gy, bool), W, H)
    f = orc.render_fwd(b["ranges"], b["point_list"], means2D, np.array([rgb], np.float32), np.array([amap], np.float32),
                       co, np.ones(gx * gy, bool), np.array(bg, np.float32), W, H, cam.tanfovx, cam.tanfovy, geo)
    return cam, f


def test_render_single_gaussian_closed_form(orc):
    W, H = 48, 32
    mean, conic, o, rgb, bg = (20.25, 11.5), (0.05, 0.01, 0.08), 0.8, (0.2, 0.6, 0.9), (0.1, 0.3, 0.5)
    amap = (0.0, 0.0, 1.0, 1.0, 7.0)  # planar Gaussian facing the camera at plane distance 7
    cam, f = _one_gaussian(orc, mean, conic, o, rgb, amap, bg, W, H)
    ys, xs = np.mgrid[0:H, 0:W].astype(np.float64)
    dx, dy = mean[0] - xs, mean[1] - ys
    power = -0.5 * (conic[0] * dx * dx + conic[2] * dy * dy) - conic[1] * dx * dy
    alpha = np.minimum(0.99, o * np.exp(power))
    alpha[alpha < 1 / 255] = 0
    for ch in range(3):
        np.testing.assert_allclose(f["color"][ch], rgb[ch] * alpha + (1 - alpha) * bg[ch], atol=2e-6)
    np.testing.assert_allclose(f["final_T"], 1 - alpha, atol=2e-6)
    np.testing.assert_allclose(f["out_all_map"][3], 1 - f["final_T"], atol=1e-6)  # alpha channel when all_map[:,3] = 1
    assert np.array_equal(f["n_contrib"], (alpha > 0).astype(np.uint32))
    assert np.array_equal(f["n_contrib2loss"], f["n_contrib"])
    # plane depth: distance / (-n . ray) with n = (0,0,1)  ->  -7 alpha / (alpha + 1e-8)
    hit = alpha > 0
    np.testing.assert_allclose(f["out_plane_depth"][0][hit], -7.0, rtol=1e-5)
    assert f["out_observe"][0] == int(hit.sum())  # T = 1 > 0.5 for every contributing pixel
    assert f["n_render"].sum() == ((W + 15) // 16) * ((H + 15) // 16)  # radius 200 covers every tile


def test_render_depth_order_and_termination(orc):
    """Two coincident opaque-ish Gaussians: the nearer one is blended first; a stack of opaque Gaussians
    stops at T < 1e-4 and later ones do not count."""
    W, H = 16, 16
    cam = _cam(W, H)
    n = 12
    means2D = np.tile(np.array([[8.0, 8.0]], np.float32), (n, 1))
    co = np.tile(np.array([[1e-4, 0.0, 1e-4, 0.8]], np.float32), (n, 1))
    depths = np.arange(n, 0, -1).astype(np.float32)  # index n-1 is nearest
    rgb = np.zeros((n, 3), np.float32)
    rgb[:, 0] = np.arange(n) / n
    b = orc.bin_and_sort(np.full(n, 50, np.int32), means2D, depths, np.ones(1, bool), W, H)
    assert np.array_equal(b["point_list"], np.arange(n - 1, -1, -1))
    f = orc.render_fwd(b["ranges"], b["point_list"], means2D, rgb, np.zeros((n, 5), np.float32), co, np.ones(1, bool),
                       np.zeros(3, np.float32), W, H, cam.tanfovx, cam.tanfovy, True)
    a = 0.8  # at the centre pixel (8,8) the exponent is 0
    T, col, cnt = 1.0, 0.0, 0
    for k in range(n - 1, -1, -1):
        if T * (1 - a) < 1e-4:
            break
        col += rgb[k, 0] * a * T
        T *= 1 - a
        cnt += 1
    assert cnt == 5  # 0.2^5 = 3.2e-4 is kept, 0.2^6 = 6.4e-5 stops the pixel
    assert f["n_contrib"][8, 8] == cnt and f["n_contrib2loss"][8, 8] == cnt
    np.testing.assert_allclose(f["color"][0, 8, 8], col, rtol=1e-5)
    np.testing.assert_allclose(f["final_T"][8, 8], T, rtol=1e-5)
    # out_observe counts pixels where T > 0.5 before blending: only the first (nearest) Gaussian
    assert f["out_observe"][n - 1] == 256 and f["out_observe"][: n - 1].sum() == 0


@pytest.mark.parametrize("seed,geo", [(0, True), (1, True), (2, False)])
def test_render_forward_backward_match_autograd(orc, seed, geo):
    W, H, P = 64, 48, 150
    cam = _cam(W, H)
    gen = torch.Generator().manual_seed(seed)
    means2D = torch.rand(P, 2, generator=gen, dtype=torch.float64) * torch.tensor([W, H]) - 0.5
    s = torch.rand(P, generator=gen, dtype=torch.float64) * 6 + 1.5
    ang = torch.rand(P, generator=gen, dtype=torch.float64) * math.pi
    ecc = torch.rand(P, generator=gen, dtype=torch.float64) * 0.6 + 0.4
    ca, sa = torch.cos(ang), torch.sin(ang)
    ia, ib = 1 / s ** 2, 1 / (s * ecc) ** 2
    conic = torch.stack([ca * ca * ia + sa * sa * ib, ca * sa * (ia - ib), sa * sa * ia + ca * ca * ib], -1)
    opac = torch.rand(P, 1, generator=gen, dtype=torch.float64) * 0.9 + 0.05
    co = torch.cat([conic, opac], 1)
    rgb = torch.rand(P, 3, generator=gen, dtype=torch.float64)
    # camera-facing normals keep the plane-depth denominator (n . ray) away from zero, so the check is
    # well conditioned in fp32
    amap = torch.randn(P, 5, generator=gen, dtype=torch.float64)
    amap[:, :2] *= 0.2
    amap[:, 2] = 1.0
    amap[:, :3] = torch.nn.functional.normalize(amap[:, :3], dim=-1)
    amap[:, 3] = 1.0
    amap[:, 4] = amap[:, 4].abs() + 1.0
    depths = torch.rand(P, generator=gen) * 10 + 1
    radii = torch.ceil(3 * s).int()
    bg = torch.tensor([0.3, 0.1, 0.7], dtype=torch.float64)
    gx, gy = orc.tile_grid(W, H)
    cl = np.ones(gx * gy, bool)
    f32 = lambda t: t.detach().float().numpy()
    b = orc.bin_and_sort(radii.numpy(), f32(means2D), depths.numpy(), cl, W, H)
    fo = orc.render_fwd(b["ranges"], b["point_list"], f32(means2D), f32(rgb), f32(amap), f32(co), cl, f32(bg), W, H,
                        cam.tanfovx, cam.tanfovy, geo)
    leaves = [t.clone().requires_grad_(True) for t in (means2D, co, rgb, amap)]
    ft = tr.render(leaves[0], leaves[1], leaves[2], leaves[3], b["ranges"], b["point_list"], bg, W, H, cam.tanfovx,
                   cam.tanfovy, geo)
    assert np.array_equal(fo["n_contrib"], ft["n_contrib"].numpy().astype(np.uint32))
    np.testing.assert_allclose(fo["color"], ft["color"].detach().numpy(), atol=3e-6)
    np.testing.assert_allclose(fo["final_T"], ft["final_T"].detach().numpy(), atol=3e-6)
    if geo:
        np.testing.assert_allclose(fo["out_all_map"], ft["out_all_map"].detach().numpy(), atol=2e-5)
        pd_ref = ft["out_plane_depth"].detach().numpy()
        np.testing.assert_allclose(fo["out_plane_depth"], pd_ref, rtol=1e-4, atol=1e-4)
    # final_T equals the product of (1 - alpha) of the blended Gaussians; sum over tiles of range lengths = instances
    assert fo["n_render"].sum() == b["num_rendered"]
    assert fo["out_observe"].sum() <= fo["n_contrib2loss"].sum()
    # backward
    gpix = torch.randn(3, H, W, generator=gen, dtype=torch.float64)
    gmap = torch.randn(5, H, W, generator=gen, dtype=torch.float64)
    gdep = torch.randn(1, H, W, generator=gen, dtype=torch.float64)
    loss = (ft["color"] * gpix).sum()
    if geo:
        loss = loss + (ft["out_all_map"] * gmap).sum() + (ft["out_plane_depth"] * gdep).sum()
    loss.backward()
    bo = orc.render_bwd(b["ranges"], b["point_list"], f32(means2D), f32(co), f32(rgb), f32(amap), fo["out_all_map"],
                        fo["final_T"], fo["n_contrib"], cl, f32(bg), f32(gpix), f32(gmap), f32(gdep), W, H, cam.tanfovx,
                        cam.tanfovy, geo)
    # the reference reports the mean2D gradient per NDC unit: pixel gradient times (W/2, H/2) (backward.cu:443-444)
    gm = leaves[0].grad.numpy() * np.array([0.5 * W, 0.5 * H])
    assert _rel(bo["dL_dmeans2D"][:, :2], gm) <= 1e-4
    assert (bo["dL_dmeans2D"][:, 2] == 0).all() and (bo["dL_dmeans2D_abs"][:, 2] == 0).all()
    # off-diagonal conic gradient is emitted at half weight (see test_preprocess_backward_matches_autograd)
    assert _rel(bo["dL_dconic_opacity"], leaves[1].grad.numpy() * np.array([1.0, 0.5, 1.0, 1.0])) <= 1e-4
    assert (bo["dL_dconic"][:, 2] == 0).all()
    assert _rel(bo["dL_dcolors"], leaves[2].grad.numpy()) <= 1e-4
    if geo:
        assert _rel(bo["dL_dall_map"], leaves[3].grad.numpy()) <= 1e-4
    else:
        assert (bo["dL_dall_map"] == 0).all()
    assert (bo["dL_dmeans2D_abs"][:, :2] >= np.abs(bo["dL_dmeans2D"][:, :2]) * (1 - 1e-5) - 1e-7).all()


@pytest.mark.parametrize("seed,geo", [(3, True), (4, False)])
def test_render_backward_abs_gradient_is_a_sum_of_per_pixel_magnitudes(orc, seed, geo):
    """dL_dmeans2D_abs (backward.cu:553-554) adds up, pixel by pixel, the magnitude of that pixel's own
    contribution to the mean2D gradient.  Pinned by differentiating every pixel's loss term on its own
    (float64 autograd through torch_ref.render) and summing the magnitudes; upstream gradients of mixed sign
    make the pixels' contributions cancel, so taking the magnitude of the finished sum instead gives a
    different number, which the last lines check."""
    W = H = 16
    P = 30
    cam = _cam(W, H)
    gen = torch.Generator().manual_seed(seed)
    means2D = torch.rand(P, 2, generator=gen, dtype=torch.float64) * 18.0 - 1.0
    s = torch.rand(P, generator=gen, dtype=torch.float64) * 3 + 1.5
    ang = torch.rand(P, generator=gen, dtype=torch.float64) * math.pi
    ecc = torch.rand(P, generator=gen, dtype=torch.float64) * 0.6 + 0.4
    ca, sa = torch.cos(ang), torch.sin(ang)
    ia, ib = 1 / s ** 2, 1 / (s * ecc) ** 2
    conic = torch.stack([ca * ca * ia + sa * sa * ib, ca * sa * (ia - ib), sa * sa * ia + ca * ca * ib], -1)
    co = torch.cat([conic, torch.rand(P, 1, generator=gen, dtype=torch.float64) * 0.6 + 0.05], 1)
    rgb = torch.rand(P, 3, generator=gen, dtype=torch.float64)
    amap = torch.randn(P, 5, generator=gen, dtype=torch.float64)
    amap[:, :2] *= 0.2
    amap[:, 2] = 1.0
    amap[:, :3] = torch.nn.functional.normalize(amap[:, :3], dim=-1)
    amap[:, 3] = 1.0
    amap[:, 4] = amap[:, 4].abs() + 1.0
    depths = torch.rand(P, generator=gen) * 10 + 1
    radii = torch.ceil(3 * s).int()
    bg = torch.tensor([0.3, 0.1, 0.7], dtype=torch.float64)
    cl = np.ones(1, bool)
    f32 = lambda t: t.detach().float().numpy()
    b = orc.bin_and_sort(radii.numpy(), f32(means2D), depths.numpy(), cl, W, H)
    fo = orc.render_fwd(b["ranges"], b["point_list"], f32(means2D), f32(rgb), f32(amap), f32(co), cl, f32(bg), W, H,
                        cam.tanfovx, cam.tanfovy, geo)
    gpix = torch.randn(3, H, W, generator=gen, dtype=torch.float64)
    gmap = torch.randn(5, H, W, generator=gen, dtype=torch.float64)
    gdep = torch.randn(1, H, W, generator=gen, dtype=torch.float64)
    m = means2D.clone().requires_grad_(True)
    ft = tr.render(m, co, rgb, amap, b["ranges"], b["point_list"], bg, W, H, cam.tanfovx, cam.tanfovy, geo)
    assert np.array_equal(fo["n_contrib"], ft["n_contrib"].numpy().astype(np.uint32))
    per_pixel = (ft["color"] * gpix).sum(0)
    if geo:
        per_pixel = per_pixel + (ft["out_all_map"] * gmap).sum(0) + (ft["out_plane_depth"] * gdep).sum(0)
    scale = torch.tensor([0.5 * W, 0.5 * H], dtype=torch.float64)
    sum_of_abs = torch.zeros(P, 2, dtype=torch.float64)
    plain_sum = torch.zeros(P, 2, dtype=torch.float64)
    for y in range(H):
        for x in range(W):
            (gp,) = torch.autograd.grad(per_pixel[y, x], m, retain_graph=True)
            sum_of_abs += (gp * scale).abs()
            plain_sum += gp * scale
    bo = orc.render_bwd(b["ranges"], b["point_list"], f32(means2D), f32(co), f32(rgb), f32(amap), fo["out_all_map"],
                        fo["final_T"], fo["n_contrib"], cl, f32(bg), f32(gpix), f32(gmap), f32(gdep), W, H, cam.tanfovx,
                        cam.tanfovy, geo)
    assert _rel(bo["dL_dmeans2D"][:, :2], plain_sum.numpy()) <= 1e-4
    assert _rel(bo["dL_dmeans2D_abs"][:, :2], sum_of_abs.numpy()) <= 1e-4
    assert (bo["dL_dmeans2D_abs"][:, 2] == 0).all()
    # the case tells the two readings apart: the magnitude of the finished sum is far from the sum of magnitudes
    assert _rel(np.abs(bo["dL_dmeans2D"][:, :2]), sum_of_abs.numpy()) > 0.2


def test_render_masked_tiles_are_untouched(orc):
    g, cams = gs_scenes.make_scene(0, P=3000)
    cam = cams[0]
    W, H = cam.image_width, cam.image_height
    o = _pre(orc, g, cam)
    gx, gy = orc.tile_grid(W, H)
    cl = np.ones((gy, gx), bool)
    cl[:, : gx // 2] = False
    b = orc.bin_and_sort(o["radii"], o["means2D"], o["depths"], cl.ravel(), W, H)
    assert (b["ranges"].reshape(gy, gx, 2)[:, : gx // 2] == 0).all()
    am = gs_scenes.build_all_map(g["means3D"], g["scales"], g["rotations"], cam).numpy()
    f = orc.render_fwd(b["ranges"], b["point_list"], o["means2D"], o["rgb"], am, o["conic_opacity"], cl.ravel(),
                       np.ones(3, np.float32), W, H, cam.tanfovx, cam.tanfovy)
    half = (gx // 2) * 16
    assert (f["color"][:, :, :half] == 0).all() and (f["color"][:, :, half:] > 0).any()
    assert (f["n_consider"].reshape(gy, gx)[:, : gx // 2] == 0).all()
    # per-tile statistics are plain sums
    nc = f["n_contrib"].astype(np.int64)
    pad = np.zeros((gy * 16, gx * 16), np.int64)
    pad[:H, :W] = nc
    sums = pad.reshape(gy, 16, gx, 16).sum(axis=(1, 3))
    assert np.array_equal(f["n_consider"].reshape(gy, gx)[:, gx // 2:], sums[:, gx // 2:])


# ---------------------------------------------------------------------- knn --

def test_morton_known_answers(orc):
    mn, mx = np.zeros(3, np.float32), np.ones(3, np.float32)
    assert orc.morton([1, 0, 0], mn, mx) == 0x09249249          # prepMorton(1023)
    assert orc.morton([0, 1, 0], mn, mx) == 0x09249249 << 1
    assert orc.morton([0, 0, 1], mn, mx) == 0x09249249 << 2
    assert orc.morton([1, 1, 1], mn, mx) == 0x3FFFFFFF
    assert orc.morton([0, 0, 0], mn, mx) == 0
    assert orc.morton([0.5, 0, 0], mn, mx) == sum(1 << (3 * b) for b in range(10) if (511 >> b) & 1)


@pytest.mark.parametrize("P,kind", [(5, "u"), (1500, "u"), (6000, "pos"), (6000, "line")])
def test_knn_against_brute_force(orc, P, kind):
    from scipy.spatial import cKDTree
    rng = np.random.default_rng(P)
    if kind == "u":
        pts = rng.uniform(-5, 5, (P, 3))
    elif kind == "pos":
        pts = rng.uniform(10, 12, (P, 3))  # bounding box reduction starts from 0: codes use a tenth of the range
    else:
        pts = np.stack([np.linspace(0, 100, P), np.zeros(P), np.zeros(P)], 1) + rng.normal(0, 1e-3, (P, 3))
    pts = pts.astype(np.float32)
    got = orc.knn_dist2(pts)
    p64 = pts.astype(np.float64)
    d, _ = cKDTree(p64).query(p64, k=4)
    np.testing.assert_allclose(got, (d[:, 1:] ** 2).mean(1), rtol=3e-5, atol=1e-12)


# ---------------------------------------------------------------- all_map --

def _all_map_case(P=4000, seed=5):
    import gs_scenes
    g, cams = gs_scenes.make_scene(0, P=P, n_views=1, seed=seed)
    return g, cams[0]


def test_all_map_forward_matches_float64_torch_and_closed_form(orc):
    import gs_scenes
    g, cam = _all_map_case()

    class C64:
        world_view_transform = cam.world_view_transform.double()
        camera_center = cam.camera_center.double()
    ref = gs_scenes.build_all_map(g["means3D"].double(), g["scales"].double(), g["rotations"].double(), C64).numpy()
    o = orc.all_map_fwd(g["means3D"].numpy(), g["scales"].numpy(), g["rotations"].numpy(),
                        cam.world_view_transform.numpy(), cam.camera_center.numpy())
    assert np.abs(o[:, :3] - ref[:, :3]).max() <= 2e-6
    assert np.all(o[:, 3] == 1.0)
    assert np.abs(o[:, 4] - ref[:, 4]).max() <= 1e-5 * max(1.0, np.abs(ref[:, 4]).max())
    # closed form: identity rotation, smallest scale along z, camera = identity at the origin looking at +z
    m = np.array([[0.5, -0.25, 4.0]], np.float32)
    s = np.array([[0.3, 0.2, 0.1]], np.float32)
    q = np.array([[2.0, 0.0, 0.0, 0.0]], np.float32)  # unnormalised on purpose
    V = np.eye(4, dtype=np.float32)
    o1 = orc.all_map_fwd(m, s, q, V, np.zeros(3, np.float32))
    # normal = +z flipped towards the camera at the origin -> (0,0,-1); distance = |n . p| = 4
    assert np.allclose(o1[0], [0.0, 0.0, -1.0, 1.0, 4.0], atol=1e-6)
    # smallest scale along x, rotation of 90 degrees about z maps the x axis to +y
    q90 = np.array([[np.sqrt(0.5), 0.0, 0.0, np.sqrt(0.5)]], np.float32)
    o2 = orc.all_map_fwd(m, np.array([[0.1, 0.2, 0.3]], np.float32), q90, V, np.zeros(3, np.float32))
    # n = +y; n . (cam - m) = 0.25 > 0: kept; distance = |-0.25|
    assert np.allclose(o2[0], [0.0, 1.0, 0.0, 1.0, 0.25], atol=1e-6)


def test_all_map_backward_matches_float64_autograd(orc):
    import gs_scenes
    g, cam = _all_map_case(seed=6)

    class C64:
        world_view_transform = cam.world_view_transform.double()
        camera_center = cam.camera_center.double()
    m = g["means3D"].double().requires_grad_(True)
    q = (g["rotations"].double() * 1.7).requires_grad_(True)  # away from unit length: exercises normalize
    out = gs_scenes.build_all_map(m, g["scales"].double(), q, C64)
    go = torch.randn(out.shape, generator=torch.Generator().manual_seed(2), dtype=torch.float64)
    (out * go).sum().backward()
    dm, dq = orc.all_map_bwd(g["means3D"].numpy(), g["scales"].numpy(), (g["rotations"] * 1.7).numpy(),
                             cam.world_view_transform.numpy(), cam.camera_center.numpy(), go.float().numpy())
    rel = lambda a, b: np.linalg.norm(a - b) / np.linalg.norm(b)
    assert rel(dm, m.grad.numpy()) <= 1e-6
    assert rel(dq, q.grad.numpy()) <= 1e-6
    # the rotation gradient is orthogonal to the quaternion (the output does not depend on its length)
    assert np.abs((dq * (g["rotations"] * 1.7).numpy()).sum(1)).max() <= 1e-4 * np.abs(dq).max()


# ------------------------------------------------------------------- Adam --

def test_adam_step_matches_torch_optim_adam(orc):
    """Library routine: torch.optim.Adam on the CPU, five steps, two parameter groups with their own lr."""
    gen = torch.Generator().manual_seed(11)
    shapes, lrs = [(1000, 3), (257,)], [1.6e-4, 5e-3]
    ps = [torch.randn(s, generator=gen) for s in shapes]
    tp = [p.clone().requires_grad_(True) for p in ps]
    opt = torch.optim.Adam([{"params": [tp[0]], "lr": lrs[0]}, {"params": [tp[1]], "lr": lrs[1]}], lr=0.0, eps=1e-15)
    mine = [(p.numpy().copy(), np.zeros(s, np.float32), np.zeros(s, np.float32)) for p, s in zip(ps, shapes)]
    for step in range(1, 6):
        grads = [torch.randn(s, generator=gen) * (10.0 ** (step - 3)) for s in shapes]
        for p, g in zip(tp, grads):
            p.grad = g.clone()
        opt.step()
        mine = [orc.adam_step(p, g.numpy(), m, v, lr, step) for (p, m, v), g, lr in zip(mine, grads, lrs)]
        for (p, m, v), t, p0 in zip(mine, tp, ps):
            st = opt.state[t]
            rel = lambda a, b: np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)
            assert rel(m, st["exp_avg"].numpy()) <= 1e-6
            assert rel(v, st["exp_avg_sq"].numpy()) <= 1e-6
            assert rel(p - p0.numpy(), t.detach().numpy() - p0.numpy()) <= 1e-5
    # first step of Adam moves every element with a non-zero gradient by lr (textbook property)
    p1, _, _ = orc.adam_step(np.zeros(4, np.float32), np.array([3.0, -2.0, 1e-3, 0.0], np.float32),
                             np.zeros(4, np.float32), np.zeros(4, np.float32), 0.01, 1)
    assert np.allclose(p1, [-0.01, 0.01, -0.01, 0.0], rtol=1e-5, atol=0)
    # grad_scale = 1/bsz is the same as dividing the gradient first
    a = orc.adam_step(ps[0].numpy(), grads[0].numpy(), mine[0][1], mine[0][2], 1e-3, 7, grad_scale=0.25)
    b = orc.adam_step(ps[0].numpy(), grads[0].numpy() * np.float32(0.25), mine[0][1], mine[0][2], 1e-3, 7)
    assert all(np.array_equal(x, y) for x, y in zip(a, b))


# ------------------------------------------------- densification statistics --

def _stats_case(A=300, k=5, seed=0, p_vis=0.6, p_sel=0.7, p_flt=0.8):
    gen = torch.Generator().manual_seed(seed)
    vis = torch.rand(A, generator=gen) < p_vis
    V = int(vis.sum())
    sel = torch.rand(V * k, generator=gen) < p_sel
    S = int(sel.sum())
    flt = torch.rand(S, generator=gen) < p_flt
    grad = torch.randn(S, 3, generator=gen)
    opacity = torch.randn(V * k, 1, generator=gen)
    acc = [torch.rand(A, 1, generator=gen), torch.rand(A, 1, generator=gen).round(),
           torch.rand(A * k, 1, generator=gen), torch.rand(A * k, 1, generator=gen).round()]
    return vis, sel, flt, grad, opacity, acc


def _stats_by_mask_indexing(acc, k, grad, opacity, flt, sel, vis):
    """The same update through torch's boolean-mask gathers and scatters (library semantics of x[mask] = y)."""
    oa, ad, ga, dn = [t.clone() for t in acc]
    temp = opacity.clone().view(-1)
    temp[temp < 0] = 0
    oa[vis] += temp.view(-1, k).sum(dim=1, keepdim=True)
    ad[vis] += 1
    vis_rep = vis.unsqueeze(1).repeat(1, k).view(-1)
    combined = torch.zeros(ga.shape[0], dtype=torch.bool)
    combined[vis_rep] = sel
    temp_mask = combined.clone()
    combined[temp_mask] = flt
    ga[combined] += torch.norm(grad[flt, :2], dim=-1, keepdim=True)
    dn[combined] += 1
    return oa, ad, ga, dn


@pytest.mark.parametrize("seed,p", [(0, (0.6, 0.7, 0.8)), (1, (1.0, 1.0, 1.0)), (2, (0.05, 0.3, 0.5)), (3, (0.5, 0.0, 0.5))])
def test_training_stats_matches_mask_indexing(orc, seed, p):
    vis, sel, flt, grad, opacity, acc = _stats_case(seed=seed, p_vis=p[0], p_sel=p[1], p_flt=p[2])
    ref = _stats_by_mask_indexing(acc, 5, grad, opacity, flt, sel, vis)
    got = orc.training_stats(acc[0].numpy(), acc[1].numpy(), acc[2].numpy(), acc[3].numpy(), 5, grad.numpy(),
                             opacity.numpy(), flt.numpy(), sel.numpy(), vis.numpy())
    for g, r in zip(got, ref):
        assert np.allclose(g, r.numpy().ravel(), rtol=1e-6, atol=1e-7)
    # counters move by whole numbers, and only where the chain of masks says so
    assert np.array_equal(got[1] - acc[1].numpy().ravel(), vis.numpy().astype(np.float32))
    assert int((got[3] - acc[3].numpy().ravel()).sum()) == int(flt.sum())


# ------------------------------------------------------------- L1 + SSIM --

def _ssim_ref64(a, b, mask, window):
    """The reference statements (utils/loss_utils.py:97-132) with torch's conv2d in float64."""
    import torch.nn.functional as F
    Cn = a.shape[0]
    w1 = torch.tensor(window).double()
    w = (w1[:, None] @ w1[None, :]).expand(Cn, 1, 11, 11).contiguous()
    conv = lambda t: F.conv2d(t[None], w, padding=5, groups=Cn)[0]
    mu1, mu2 = conv(a), conv(b)
    s1, s2, s12 = conv(a * a) - mu1 ** 2, conv(b * b) - mu2 ** 2, conv(a * b) - mu1 * mu2
    m = ((2 * mu1 * mu2 + 0.01 ** 2) * (2 * s12 + 0.03 ** 2)) / ((mu1 ** 2 + mu2 ** 2 + 0.01 ** 2) * (s1 + s2 + 0.03 ** 2))
    return torch.abs(a - b) * mask[None], m * mask[None]


def test_ssim_window_is_create_window(orc):
    w = orc.ssim_window()
    assert w.dtype == np.float32 and w.shape == (11,)
    assert abs(float(w.sum()) - 1.0) < 1e-6 and np.array_equal(w, w[::-1]) and w.argmax() == 5
    assert abs(w[5] / w[4] - np.exp(1.0 / 4.5)) < 1e-6  # sigma = 1.5


def test_ssim_l1_forward_and_backward_match_float64_torch(orc):
    gen = torch.Generator().manual_seed(0)
    Cn, H, W = 3, 37, 52  # not multiples of the window or of any block size; borders matter
    a = torch.rand(Cn, H, W, generator=gen)
    b = (a + 0.2 * torch.randn(Cn, H, W, generator=gen)).clamp(0, 1)
    mask = torch.rand(H, W, generator=gen) < 0.7
    ad = a.double().requires_grad_(True)
    l1r, sr = _ssim_ref64(ad, b.double(), mask, orc.ssim_window())
    l1, ss = orc.ssim_l1_fwd(a.numpy(), b.numpy(), mask.numpy())
    assert np.abs(l1 - l1r.detach().numpy()).max() <= 1e-7
    assert np.abs(ss - sr.detach().numpy()).max() <= 2e-5
    g1, g2 = torch.randn(Cn, H, W, generator=gen), torch.randn(Cn, H, W, generator=gen)
    ((l1r * g1.double()).sum() + (sr * g2.double()).sum()).backward()
    d = orc.ssim_l1_bwd(a.numpy(), b.numpy(), mask.numpy(), g1.numpy(), g2.numpy())
    assert np.linalg.norm(d - ad.grad.numpy()) / np.linalg.norm(ad.grad.numpy()) <= 1e-5


def test_ssim_closed_forms(orc):
    H, W = 30, 40
    a = torch.rand(3, H, W, generator=torch.Generator().manual_seed(1)).numpy()
    l1, ss = orc.ssim_l1_fwd(a, a, None)
    assert np.all(l1 == 0) and np.all(ss == 1.0)         # an image against itself
    ca, cb = np.full((1, H, W), 0.3, np.float32), np.full((1, H, W), 0.6, np.float32)
    l1, ss = orc.ssim_l1_fwd(ca, cb, None)
    assert np.allclose(l1, 0.3, atol=1e-7)
    want = (2 * 0.3 * 0.6 + 1e-4) / (0.3 ** 2 + 0.6 ** 2 + 1e-4)   # constants: no variance, full window inside
    assert np.abs(ss[0, 5:-5, 5:-5] - want).max() <= 1e-4
    m = np.zeros((H, W), bool)
    m[3:9, 4:20] = True
    l1m, ssm = orc.ssim_l1_fwd(ca, cb, m)
    assert np.all(ssm[0][~m] == 0) and np.all(l1m[0][~m] == 0) and np.array_equal(ssm[0][m], ss[0][m])


# ------------------------------------------------- neural-Gaussian generation --

def _anchor_scene_np(N, k, seed):
    s = gs_scenes.make_anchor_scene(N, k, seed)
    n = lambda t: t.numpy()
    mlps = [tuple(n(x) for x in m) for m in s["mlps"]]
    return s, (n(s["anchor"]), n(s["feat"]), n(s["offsets"]), n(s["scaling"]), n(s["campos"]), mlps)


@pytest.mark.parametrize("N,k,seed", [(257, 10, 0), (64, 5, 1), (1, 10, 2)])
def test_neural_gaussians_forward_matches_float64_torch(orc, N, k, seed):
    s, args = _anchor_scene_np(N, k, seed)
    got = orc.neural_gaussians_fwd(*args)
    d = lambda t: t.double()
    want = gs_scenes.neural_gaussians_torch(d(s["anchor"]), d(s["feat"]), d(s["offsets"]), d(s["scaling"]),
                                            d(s["campos"]), [tuple(d(x) for x in m) for m in s["mlps"]])
    # the selection is a threshold on a float32 value: equal unless an opacity sits within rounding of zero
    wmask = want[6].numpy()
    near = np.abs(want[5].numpy().ravel()) < 1e-6
    assert (got[6] == wmask)[~near].all()
    if (got[6] == wmask).all():
        for g, w in zip(got[:6], want[:6]):
            assert g.shape == tuple(w.shape)
            assert _rel(g, w.numpy()) < 2e-6
    assert got[0].shape[0] == int(got[6].sum()) and 0 < got[6].sum() < N * k or N == 1
    # rotations are unit quaternions, opacities are the positive dense ones in slot order
    assert np.allclose(np.linalg.norm(got[4], axis=1), 1.0, atol=1e-6)
    assert np.array_equal(got[2].ravel(), got[5].ravel()[got[6]])


def test_neural_gaussians_known_case(orc):
    """Zero weights: every output is its bias through the activation; one offset switched off by a negative bias."""
    N, k = 3, 4
    s, (anchor, feat, offsets, scaling, campos, mlps) = _anchor_scene_np(N, k, 5)
    z = lambda a: np.zeros_like(a)
    b_op = np.array([0.5, -0.5, 0.25, 1.0], np.float32)
    b_col = np.linspace(-1, 1, 3 * k).astype(np.float32)
    b_cov = np.tile(np.array([0.0, 1.0, -1.0, 2.0, 0.0, 0.0, 0.0], np.float32), k)
    mlps = [(z(mlps[0][0]), z(mlps[0][1]), z(mlps[0][2]), b_op), (z(mlps[1][0]), z(mlps[1][1]), z(mlps[1][2]), b_col),
            (z(mlps[2][0]), z(mlps[2][1]), z(mlps[2][2]), b_cov)]
    xyz, col, op, sc, rot, nop, mask = orc.neural_gaussians_fwd(anchor, feat, offsets, scaling, campos, mlps)
    assert mask.reshape(N, k).tolist() == [[True, False, True, True]] * N
    keep = [0, 2, 3]
    assert np.allclose(op.reshape(N, 3), np.tanh(b_op[keep].astype(np.float64)), rtol=1e-6)
    sig = lambda v: 1 / (1 + np.exp(-v.astype(np.float64)))
    assert np.allclose(col.reshape(N, 3, 3), sig(b_col.reshape(k, 3)[keep]), rtol=1e-6)
    assert np.allclose(rot, [1.0, 0.0, 0.0, 0.0])
    assert np.allclose(sc.reshape(N, 3, 3), scaling[:, None, 3:] * sig(b_cov[:3])[None, None, :], rtol=1e-6)
    assert np.allclose(xyz.reshape(N, 3, 3), anchor[:, None, :] + offsets[:, keep, :] * scaling[:, None, :3], rtol=1e-6)


@pytest.mark.parametrize("N,k,seed", [(193, 10, 3), (50, 5, 4)])
def test_neural_gaussians_backward_matches_float64_autograd(orc, N, k, seed):
    s, args = _anchor_scene_np(N, k, seed)
    fwd = orc.neural_gaussians_fwd(*args)
    S = fwd[0].shape[0]
    gen = torch.Generator().manual_seed(seed)
    ups = [torch.randn(S, c, generator=gen) for c in (3, 3, 1, 3, 4)]
    got = orc.neural_gaussians_bwd(*args, *[u.numpy() for u in ups])
    leaf = lambda t: t.double().requires_grad_(True)
    anchor, feat, offsets, scaling = leaf(s["anchor"]), leaf(s["feat"]), leaf(s["offsets"]), leaf(s["scaling"])
    mlps = [tuple(leaf(x) for x in m) for m in s["mlps"]]
    out = gs_scenes.neural_gaussians_torch(anchor, feat, offsets, scaling, s["campos"].double(), mlps)
    assert np.array_equal(out[6].numpy(), fwd[6])
    loss = sum((o * u.double()).sum() for o, u in zip(out[:5], ups))
    loss.backward()
    for name, g, w in zip(("anchor", "feat", "offsets", "scaling"), got[:4], (anchor, feat, offsets, scaling)):
        assert _rel(g, w.grad.numpy()) < 1e-5, name
    flat = [x for m in mlps for x in m]
    for i, (g, w) in enumerate(zip(got[4], flat)):
        assert g.shape == tuple(w.shape)
        assert _rel(g, w.grad.numpy()) < 1e-5, i


def _prog(N, seed):
    """Per-anchor opacity factor as dist2level 'progressive' builds it: a ratio in (0, 1), 1 outside the transition
    mask, and a few anchors switched off altogether (ratio 0)."""
    gen = torch.Generator().manual_seed(100 + seed)
    prog = torch.rand(N, 1, generator=gen) * 0.98 + 0.01
    prog[torch.rand(N, generator=gen) < 0.4] = 1.0
    prog[torch.rand(N, generator=gen) < 0.1] = 0.0
    return prog


@pytest.mark.parametrize("N,k,seed", [(193, 10, 6), (40, 5, 7)])
def test_neural_gaussians_progressive_factor_matches_float64_torch(orc, N, k, seed):
    """The factor scales the dense opacity and the selected one, switches an anchor with ratio 0 off, and reaches
    the opacity MLP's gradients and nothing else (gaussian_renderer/__init__.py:844-848)."""
    s, args = _anchor_scene_np(N, k, seed)
    prog = _prog(N, seed)
    plain = orc.neural_gaussians_fwd(*args)
    fwd = orc.neural_gaussians_fwd(*args, prog=prog.numpy())
    assert np.allclose(fwd[5].reshape(N, k), plain[5].reshape(N, k) * prog.numpy(), rtol=1e-6, atol=0)
    assert np.array_equal(fwd[6].reshape(N, k), plain[6].reshape(N, k) & (prog.numpy() > 0))
    assert not fwd[6].reshape(N, k)[prog.numpy().ravel() == 0].any()
    S = fwd[0].shape[0]
    gen = torch.Generator().manual_seed(seed)
    ups = [torch.randn(S, c, generator=gen) for c in (3, 3, 1, 3, 4)]
    got = orc.neural_gaussians_bwd(*args, *[u.numpy() for u in ups], prog=prog.numpy())
    leaf = lambda t: t.double().requires_grad_(True)
    anchor, feat, offsets, scaling = leaf(s["anchor"]), leaf(s["feat"]), leaf(s["offsets"]), leaf(s["scaling"])
    mlps = [tuple(leaf(x) for x in m) for m in s["mlps"]]
    out = gs_scenes.neural_gaussians_torch(anchor, feat, offsets, scaling, s["campos"].double(), mlps, prog.double())
    assert np.array_equal(out[6].numpy(), fwd[6])
    for g, w in zip(fwd[:6], out[:6]):
        assert _rel(g, w.detach().numpy()) < 2e-6
    loss = sum((o * u.double()).sum() for o, u in zip(out[:5], ups))
    loss.backward()
    for name, g, w in zip(("anchor", "feat", "offsets", "scaling"), got[:4], (anchor, feat, offsets, scaling)):
        assert _rel(g, w.grad.numpy()) < 1e-5, name
    flat = [x for m in mlps for x in m]
    for i, (g, w) in enumerate(zip(got[4], flat)):
        assert _rel(g, w.grad.numpy()) < 1e-5, i


@pytest.mark.parametrize("N,k,seed,flags", [(150, 10, 8, 15), (60, 5, 9, 1), (60, 4, 10, 2), (60, 3, 11, 4),
                                            (90, 10, 12, 8), (70, 6, 13, 13)])
def test_neural_gaussians_distance_and_level_inputs_match_float64_torch(orc, N, k, seed, flags):
    """add_opacity_dist / add_color_dist / add_cov_dist / add_level (gaussian_renderer/__init__.py:824-877): the
    first layers take the distance and the level as further columns; the distance carries a gradient to the anchor."""
    s = gs_scenes.make_anchor_scene(N, k, seed, input_flags=flags)
    n = lambda t: t.numpy()
    mlps_np = [tuple(n(x) for x in m) for m in s["mlps"]]
    args = (n(s["anchor"]), n(s["feat"]), n(s["offsets"]), n(s["scaling"]), n(s["campos"]), mlps_np)
    fwd = orc.neural_gaussians_fwd(*args, level=n(s["level"]), input_flags=flags)
    S = fwd[0].shape[0]
    gen = torch.Generator().manual_seed(seed)
    ups = [torch.randn(S, c, generator=gen) for c in (3, 3, 1, 3, 4)]
    got = orc.neural_gaussians_bwd(*args, *[u.numpy() for u in ups], level=n(s["level"]), input_flags=flags)
    leaf = lambda t: t.double().requires_grad_(True)
    anchor, feat, offsets, scaling = leaf(s["anchor"]), leaf(s["feat"]), leaf(s["offsets"]), leaf(s["scaling"])
    mlps = [tuple(leaf(x) for x in m) for m in s["mlps"]]
    out = gs_scenes.neural_gaussians_torch(anchor, feat, offsets, scaling, s["campos"].double(), mlps,
                                           level=s["level"].double(), input_flags=flags)
    assert np.array_equal(out[6].numpy(), fwd[6])
    for g, w in zip(fwd[:6], out[:6]):
        assert _rel(g, w.detach().numpy()) < 2e-6
    sum((o * u.double()).sum() for o, u in zip(out[:5], ups)).backward()
    for name, g, w in zip(("anchor", "feat", "offsets", "scaling"), got[:4], (anchor, feat, offsets, scaling)):
        assert _rel(g, w.grad.numpy()) < 1e-5, name
    flat = [x for m in mlps for x in m]
    for i, (g, w) in enumerate(zip(got[4], flat)):
        assert g.shape == tuple(w.shape)
        assert _rel(g, w.grad.numpy()) < 1e-5, i
    # the optional inputs matter: without them the same weights' leading columns give another result
    if flags:
        plain = orc.neural_gaussians_fwd(*args[:5], [(m[0][:, :35].copy(), m[1], m[2], m[3]) for m in mlps_np])
        same_selection = np.array_equal(plain[6], fwd[6])
        assert not (same_selection and all(np.allclose(a, b, atol=1e-4) for a, b in zip(plain[:6], fwd[:6])))


# ------------------------------------------------------ max-weight depth --

def test_max_weight_depth_known_cases(orc):
    """Closed cases: one Gaussian (its depth wherever it blends, 0 elsewhere); a faint near one in front of a strong
    far one (the far one wins where alpha_far (1 - alpha_near) > alpha_near); equal weights (the front one wins)."""
    W, H = 48, 32
    gx, gy = orc.tile_grid(W, H)
    cl = np.ones(gx * gy, bool)
    # one Gaussian
    m1 = np.array([[20.25, 11.5]], np.float32)
    co1 = np.array([[0.05, 0.01, 0.08, 0.8]], np.float32)
    b = orc.bin_and_sort(np.array([200], np.int32), m1, np.array([5.0], np.float32), cl, W, H)
    d = orc.max_weight_depth(b["ranges"], b["point_list"], m1, co1, np.array([5.0], np.float32), cl, W, H)[0]
    ys, xs = np.mgrid[0:H, 0:W].astype(np.float64)
    dx, dy = 20.25 - xs, 11.5 - ys
    alpha = 0.8 * np.exp(-0.5 * (0.05 * dx * dx + 0.08 * dy * dy) - 0.01 * dx * dy)
    sure = np.abs(alpha - 1 / 255) > 1e-6
    assert np.array_equal(d[sure], np.where(alpha >= 1 / 255, 5.0, 0.0).astype(np.float32)[sure])
    # near faint (depth 2, opacity 0.2), far strong (depth 9, opacity 0.9), both flat over the image
    m2 = np.array([[24.0, 16.0], [24.0, 16.0]], np.float32)
    flat = lambda o: [1e-7, 0.0, 1e-7, o]
    co2 = np.array([flat(0.2), flat(0.9)], np.float32)
    dep2 = np.array([2.0, 9.0], np.float32)
    b = orc.bin_and_sort(np.array([200, 200], np.int32), m2, dep2, cl, W, H)
    assert b["point_list"][:2].tolist() == [0, 1]
    d = orc.max_weight_depth(b["ranges"], b["point_list"], m2, co2, dep2, cl, W, H)[0]
    assert (d == 9.0).all()  # 0.9 * 0.8 = 0.72 > 0.2
    co2[0, 3] = 0.6  # now 0.9 * 0.4 = 0.36 < 0.6: the near one wins
    d = orc.max_weight_depth(b["ranges"], b["point_list"], m2, co2, dep2, cl, W, H)[0]
    assert (d == 2.0).all()
    co2[0, 3], co2[1, 3] = 0.5, 0.99  # weights 0.5 and 0.99 * 0.5 = 0.495 -> near; with alpha clamp 0.99
    d = orc.max_weight_depth(b["ranges"], b["point_list"], m2, co2, dep2, cl, W, H)[0]
    assert (d == 2.0).all()
    # exactly equal weights: alpha 0.5 then alpha 1.0 -> clamped to 0.99 ... use 0.5 and 0.5/(1-0.5) is not
    # representable below the clamp, so take three Gaussians 0.5, 0.5, 0.5: weights 0.5, 0.25, 0.125 -> front
    m3 = np.tile(m2[:1], (3, 1))
    co3 = np.array([flat(0.5)] * 3, np.float32)
    dep3 = np.array([3.0, 4.0, 5.0], np.float32)
    b = orc.bin_and_sort(np.full(3, 200, np.int32), m3, dep3, cl, W, H)
    d = orc.max_weight_depth(b["ranges"], b["point_list"], m3, co3, dep3, cl, W, H)[0]
    assert (d == 3.0).all()


def test_max_weight_depth_against_float64_weights(orc):
    """A random scene: the winner is the contributor whose float64 weight is largest (pixels where the two largest
    weights are within 1e-5 of each other are left out), and pixels of masked tiles stay 0."""
    g, cams = gs_scenes.make_scene(0, P=20000, n_views=1)
    cam = cams[0]
    W, H = cam.image_width, cam.image_height
    pre = _pre(orc, g, cam)
    gx, gy = orc.tile_grid(W, H)
    cl = np.ones(gx * gy, bool)
    cl[::3] = False
    b = orc.bin_and_sort(pre["radii"], pre["means2D"], pre["depths"], cl, W, H)
    got = orc.max_weight_depth(b["ranges"], b["point_list"], pre["means2D"], pre["conic_opacity"], pre["depths"], cl, W,
                               H)[0]
    ranges = b["ranges"].reshape(-1, 2)
    checked = 0
    rng = np.random.default_rng(0)
    for tile in rng.choice(gx * gy, 60, replace=False):
        ty, tx = divmod(int(tile), gx)
        ys, xs = np.mgrid[ty * 16:min(ty * 16 + 16, H), tx * 16:min(tx * 16 + 16, W)]
        if not cl[tile]:
            assert (got[ys, xs] == 0).all()
            continue
        ids = b["point_list"][ranges[tile, 0]:ranges[tile, 1]]
        if len(ids) == 0:
            assert (got[ys, xs] == 0).all()
            continue
        mu = pre["means2D"][ids].astype(np.float64)
        co = pre["conic_opacity"][ids].astype(np.float64)
        dx = mu[:, 0, None, None] - xs[None]
        dy = mu[:, 1, None, None] - ys[None]
        power = -0.5 * (co[:, 0, None, None] * dx * dx + co[:, 2, None, None] * dy * dy) - co[:, 1, None, None] * dx * dy
        alpha = np.minimum(0.99, co[:, 3, None, None] * np.exp(power))
        alpha[(power > 0) | (alpha < 1 / 255)] = 0
        Tr = np.cumprod(1 - alpha, axis=0)
        T_before = np.concatenate([np.ones_like(Tr[:1]), Tr[:-1]], axis=0)
        w = alpha * T_before
        w[Tr < 1e-4] = 0  # the Gaussian that would take T below 1e-4 and all after it do not blend
        order = np.sort(w, axis=0)
        clear = ((order[-1] - (order[-2] if len(ids) > 1 else 0)) > 1e-5) | (order[-1] == 0)
        near_stop = np.any(np.abs(Tr - 1e-4) < 1e-7, axis=0) | np.any(np.abs(alpha - 1 / 255) < 1e-7, axis=0)
        ok = clear & ~near_stop
        win = np.argmax(w, axis=0)
        want = np.where(order[-1] > 0, pre["depths"][ids][win], 0.0).astype(np.float32)
        assert np.array_equal(got[ys, xs][ok], want[ok])
        checked += int(ok.sum())
    assert checked > 5000
