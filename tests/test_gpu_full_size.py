"""Full-size checks on the GPU through properties that do not need a CPU run of the same size:
the headline workload (1 M Gaussians, 1152x864) end to end, and the radix sort at sizes where the
look-back spans hundreds of tile groups."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def H():
    import gpu_harness
    return gpu_harness


# (134 217 728 pairs on 45 bits: the "more than 100 M keys" of BASELINE config 3, whose own generator stays below)
@pytest.mark.timeout(600)
@pytest.mark.parametrize("n,end_bit", [(5_000_000, 44), (20_000_001, 45), (33_554_432, 64), (134_217_728, 45)])
def test_sort_large_is_stable_permutation(H, n, end_bit):
    g = torch.Generator(device=DEV).manual_seed(n)
    tile_bits = min(end_bit - 32, 13)
    tiles = torch.randint(0, 1 << tile_bits, (n,), generator=g, device=DEV, dtype=torch.int64)
    # few distinct depths, so equal keys are common and stability is visible
    depth = torch.randint(0, 1000, (n,), generator=g, device=DEV, dtype=torch.int64) * 4_000_037 % (1 << 32)
    keys = (tiles << 32) | depth
    vals = torch.arange(n, dtype=torch.int32, device=DEV)
    ko, vo = H.sort_pairs_u64(keys, vals, end_bit)
    # sorted by key, and by original position among equal keys: (key, value) pairs strictly increase
    dk = ko[1:] - ko[:-1]
    assert bool((dk >= 0).all())
    dv = vo[1:].to(torch.int64) - vo[:-1].to(torch.int64)
    assert bool(((dk > 0) | (dv > 0)).all())
    # a permutation that carries every value with its key
    assert bool((keys[vo.to(torch.int64)] == ko).all())
    seen = torch.zeros(n, dtype=torch.bool, device=DEV)
    seen[vo.to(torch.int64)] = True
    assert bool(seen.all())


def test_config1_full_size(H):
    """BASELINE config 1 at its real size through the operator-level functions."""
    import gs_scenes
    import gsrast_native as gn
    from diff_gaussian_rasterization import _C
    g, cams = gs_scenes.make_scene(1, n_views=1)
    cam = cams[0]
    W, Hh = cam.image_width, cam.image_height
    P = g["means3D"].shape[0]
    assert P == 1_000_000 and (W, Hh) == (1152, 864)
    d = {k: v.to(DEV) for k, v in g.items() if torch.is_tensor(v)}
    vm, pm, cp = cam.world_view_transform.to(DEV), cam.full_proj_transform.to(DEV), cam.camera_center.to(DEV)
    args = {"stats_collector": {}}

    def forward():
        _, means2D, depths, radii, cov3D, co, rgb, clamped = _C.preprocess_gaussians(
            d["means3D"], d["scales"], d["rotations"], d["shs"], d["opacities"], 1.0, vm, pm, cam.tanfovx,
            cam.tanfovy, Hh, W, 3, cp, False, False, args)
        am = gs_scenes.build_all_map(d["means3D"], d["scales"], d["rotations"], cam)
        gx, gy = (W + 15) // 16, (Hh + 15) // 16
        cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
        out = _C.render_gaussians(torch.zeros(3, device=DEV), Hh, W, means2D, depths, radii, co, rgb, cl, vm, cp,
                                  cam.tanfovx, cam.tanfovy, am, True, False, args)
        return (means2D, depths, radii, cov3D, co, rgb, clamped, am, cl), out

    pre, out = forward()
    means2D, depths, radii, cov3D, co, rgb, clamped, am, cl = pre
    R, color, n_render, n_consider, n_contrib, out_observe, oam, opd, geomB, binB, imgB = out
    T = n_render.numel()
    assert R > 1_000_000 and int(n_render.sum()) == R

    # the binning buffer: keys sorted on the compared bits, point_list consistent with the tile counts
    off = [C.c_size_t() for _ in range(5)]
    gn.check(gn.lib.gs_binning_state_layout(R, W, Hh, *[C.byref(o) for o in off]), "layout")
    base = (binB.data_ptr() + 255) // 256 * 256 - binB.data_ptr()
    point_list = binB[base + off[0].value: base + off[0].value + 4 * R].view(torch.int32)
    keys = binB[base + off[1].value: base + off[1].value + 8 * R].view(torch.int64)
    end_bit = 32 + gn.lib.gs_higher_msb(T)
    masked = keys & ((1 << end_bit) - 1)
    assert bool((masked[1:] >= masked[:-1]).all())
    tile_of = (masked >> 32)
    assert int(tile_of.max()) < T
    assert bool((torch.bincount(tile_of, minlength=T) == n_render.to(torch.int64)).all())
    goff = [C.c_size_t() for _ in range(3)]
    gn.check(gn.lib.gs_geometry_state_layout(P, *[C.byref(o) for o in goff]), "layout")
    gbase = (geomB.data_ptr() + 255) // 256 * 256 - geomB.data_ptr()
    tiles_touched = geomB[gbase + goff[0].value: gbase + goff[0].value + 4 * P].view(torch.int32)
    assert bool((torch.bincount(point_list.to(torch.int64), minlength=P) == tiles_touched.to(torch.int64)).all())
    assert bool((tiles_touched[radii == 0] == 0).all())
    # depth keys of a tile's list ascend in the order of the list (spot check on the fullest tile)
    t_big = int(n_render.argmax())
    sel = (tile_of == t_big).nonzero().squeeze(1)
    dsel = depths[point_list[sel].to(torch.int64)]
    assert bool((dsel[1:] >= dsel[:-1]).all())

    # images
    ioff = [C.c_size_t() for _ in range(5)]
    gn.check(gn.lib.gs_image_state_layout(W, Hh, *[C.byref(o) for o in ioff]), "layout")
    ibase = (imgB.data_ptr() + 255) // 256 * 256 - imgB.data_ptr()
    final_T = imgB[ibase + ioff[0].value: ibase + ioff[0].value + 4 * W * Hh].view(torch.float32)
    assert bool(torch.isfinite(color).all()) and bool(torch.isfinite(oam).all())
    assert float(final_T.min()) >= 0.0 and float(final_T.max()) <= 1.0
    assert bool((color >= 0).all())  # SH colours are clamped at 0 and the background is black
    assert int(out_observe.sum()) <= int(n_contrib.sum()) and int(n_contrib.sum()) <= int(n_consider.sum())

    # the forward pass is deterministic bit for bit
    pre2, out2 = forward()
    for a, b in zip(out[:8], out2[:8]):
        if torch.is_tensor(a):
            assert torch.equal(a, b)
        else:
            assert a == b

    # backward: repeatable to rounding of the LDS sums, and linear in the upstream gradient
    ug = gs_scenes.upstream_grads(cam)
    gc, ga, gd = ug["color"].to(DEV), ug["all_map"].to(DEV), ug["plane_depth"].to(DEV)

    def backward(scale):
        return _C.render_gaussians_backward(torch.zeros(3, device=DEV), cam.tanfovx, cam.tanfovy, oam, am, R, geomB,
                                            binB, imgB, cl, gc * scale, ga * scale, gd * scale, means2D, co, rgb,
                                            True, False, args)

    b1, b1r, b2 = backward(1.0), backward(1.0), backward(2.0)
    for x, y, z in zip(b1, b1r, b2):
        assert bool(torch.isfinite(x).all())
        nx = float(x.double().norm())
        assert float((x.double() - y.double()).norm()) <= 1e-5 * nx
        assert float((2.0 * x.double() - z.double()).norm()) <= 1e-5 * 2 * nx
    # gradients vanish exactly for Gaussians that were culled or never rendered
    dead = radii == 0
    assert float(b1[0][dead].abs().max()) == 0.0 and float(b1[3][dead].abs().max()) == 0.0
    pb = _C.preprocess_gaussians_backward(radii, cov3D, clamped, d["means3D"], d["scales"], d["rotations"], d["shs"],
                                          1.0, vm, pm, cam.tanfovx, cam.tanfovy, Hh, W, 3, cp, b1[0], b1[2], b1[3],
                                          R, False, args)
    for t in pb:
        assert bool(torch.isfinite(t).all())
    assert float(pb[3][dead].abs().max()) == 0.0  # dL/dshs of culled Gaussians


@pytest.mark.parametrize("cfg,P", [(1, 1_000_000), (3, 10_000_000)])
def test_list_routes_agree_at_full_size(H, cfg, P):
    """The per-tile lists at BASELINE sizes (config 1; config 3: 10 M Gaussians, 1920x1080, street level, lists of
    more than 8192 records) come out the same bit for bit by the radix sort over all keys (checked against numpy at
    small sizes and through its properties at large ones), by the per-tile sorts, by the per-tile radix sort from
    256 records on, and by the per-tile radix sort going block by block (3000 records) through memory."""
    import gs_scenes
    import gsrast_native as gn
    from diff_gaussian_rasterization import _C
    g, cams = gs_scenes.make_scene(cfg, P=P, n_views=1)
    cam = cams[0]
    W, Hh = cam.image_width, cam.image_height
    d = {k: v.to(DEV) for k, v in g.items() if torch.is_tensor(v)}
    vm, pm, cp = cam.world_view_transform.to(DEV), cam.full_proj_transform.to(DEV), cam.camera_center.to(DEV)
    args = {"stats_collector": {}}
    _, means2D, depths, radii, cov3D, co, rgb, clamped = _C.preprocess_gaussians(
        d["means3D"], d["scales"], d["rotations"], d["shs"], d["opacities"], 1.0, vm, pm, cam.tanfovx, cam.tanfovy,
        Hh, W, 3, cp, False, False, args)
    del d
    am = torch.zeros(P, 5, device=DEV)
    gx, gy = (W + 15) // 16, (Hh + 15) // 16
    T = gx * gy
    cl = torch.ones(gy, gx, dtype=torch.bool, device=DEV)
    results = []
    for limits in [(0, 0), (-1, -1), (256, 0), (-1, 3000)]:
        args["tile_sort_limits"] = limits
        out = _C.render_gaussians(torch.zeros(3, device=DEV), Hh, W, means2D, depths, radii, co, rgb, cl, vm, cp,
                                  cam.tanfovx, cam.tanfovy, am, False, False, args)
        R, color, n_render, binB, imgB = out[0], out[1], out[2], out[9], out[10]
        off = [C.c_size_t() for _ in range(5)]
        gn.check(gn.lib.gs_binning_state_layout(R, W, Hh, *[C.byref(o) for o in off]), "layout")
        base = (binB.data_ptr() + 255) // 256 * 256 - binB.data_ptr()
        point_list = binB[base + off[0].value: base + off[0].value + 4 * R].view(torch.int32).clone()
        keys = binB[base + off[1].value: base + off[1].value + 8 * R].view(torch.int64).clone()
        ioff = [C.c_size_t() for _ in range(5)]
        gn.check(gn.lib.gs_image_state_layout(W, Hh, *[C.byref(o) for o in ioff]), "layout")
        ibase = (imgB.data_ptr() + 255) // 256 * 256 - imgB.data_ptr()
        ranges = imgB[ibase + ioff[3].value: ibase + ioff[3].value + 8 * T].view(torch.int32).clone()
        results.append((limits, R, keys, point_list, ranges, color.clone(), n_render.clone()))
        del out, binB, imgB
    _, R0, keys0, pl0, ranges0, color0, nr0 = results[0]
    assert R0 > 1_000_000
    if cfg == 3:
        assert int(nr0.max()) > 8192  # so that the last setting really goes block by block through memory
    for limits, R, keys, pl, ranges, color, nr in results[1:]:
        assert R == R0, limits
        assert torch.equal(ranges, ranges0), limits
        assert torch.equal(keys, keys0), limits
        assert torch.equal(pl, pl0), limits
        assert torch.equal(nr, nr0) and torch.equal(color, color0), limits


def test_knn_large_against_brute_force_on_a_sample():
    """distCUDA2 on 3 M points; 512 of them checked against an exhaustive search done with torch."""
    from simple_knn._C import distCUDA2
    P = 3_000_000
    g = torch.Generator(device=DEV).manual_seed(12)
    pts = torch.rand(P, 3, generator=g, device=DEV) * torch.tensor([2000.0, 2000.0, 80.0], device=DEV)
    pts[:P // 10] = pts[:P // 10] * torch.tensor([0.05, 0.05, 1.0], device=DEV)  # a dense cluster: uneven boxes
    got = distCUDA2(pts)
    assert got.shape == (P,) and bool(torch.isfinite(got).all()) and float(got.min()) > 0.0
    q = torch.randint(0, P, (512,), generator=g, device=DEV)
    best = torch.full((512, 3), float("inf"), device=DEV)
    for s in range(0, P, 250_000):
        blk = pts[s:s + 250_000]
        d = blk[None, :, :] - pts[q][:, None, :]
        d2 = (d[..., 0] * d[..., 0] + d[..., 1] * d[..., 1]) + d[..., 2] * d[..., 2]
        own = (q[:, None] == (torch.arange(blk.shape[0], device=DEV)[None, :] + s))
        d2 = torch.where(own, torch.full_like(d2, float("inf")), d2)
        best = torch.cat([best, d2], dim=1).topk(3, dim=1, largest=False).values
    want = ((best[:, 0] + best[:, 1]) + best[:, 2]) / 3.0
    # torch may contract its multiply-adds, the search does not: equal up to the last bits of a distance
    assert float(((got[q] - want).abs() / want).max()) <= 1e-6
