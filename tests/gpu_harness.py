"""Test-side helpers that call libgsrast.so stage by stage through its C ABI
with torch GPU tensors, and run the CPU oracle on the same inputs."""
import ctypes as C

import numpy as np
import torch

import gs_scenes
import gsrast_native as gn

lib = gn.lib
DEV = "cuda:0"


def ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def dev(x, dtype=None):
    t = torch.as_tensor(np.ascontiguousarray(x)) if not torch.is_tensor(x) else x
    if dtype is not None:
        t = t.to(dtype)
    return t.contiguous().to(DEV)


def as_u32(a):
    """numpy uint32 -> int32 torch tensor on the GPU holding the same bits."""
    return dev(np.ascontiguousarray(a, np.uint32).view(np.int32))


def as_u64(a):
    return dev(np.ascontiguousarray(a, np.uint64).view(np.int64))


def np_u32(t):
    return t.cpu().numpy().view(np.uint32)


def np_u64(t):
    return t.cpu().numpy().view(np.uint64)


def grid(W, H):
    return (W + 15) // 16, (H + 15) // 16


def preprocess_fwd(g, cam, sh_mode=True, sh_degree=3, want_tiles=True, want_ddir=False):
    P = g["means3D"].shape[0]
    W, H = cam.image_width, cam.image_height
    o = dict(
        means2D=torch.empty(P, 2, device=DEV), depths=torch.empty(P, device=DEV),
        radii=torch.empty(P, dtype=torch.int32, device=DEV), cov3D=torch.empty(P, 6, device=DEV),
        conic_opacity=torch.empty(P, 4, device=DEV), rgb=torch.empty(P, 3, device=DEV),
        clamped=torch.empty(P, 3, dtype=torch.uint8, device=DEV),
        tiles_touched=torch.empty(P, dtype=torch.int32, device=DEV))
    if want_ddir:
        o["dcolor_ddir"] = torch.empty(P, 3, 3, device=DEV)
    for v in o.values():
        v.fill_(77)  # the kernel must overwrite every element
    gd = {k: dev(v) for k, v in g.items() if torch.is_tensor(v)}
    V, PM, cp = dev(cam.world_view_transform), dev(cam.full_proj_transform), dev(cam.camera_center)
    M = gd["shs"].shape[1] if sh_mode else 0
    gn.check(lib.gs_preprocess_forward(
        ptr(o["means2D"]), ptr(o["depths"]), ptr(o["radii"]), ptr(o["cov3D"]), ptr(o["conic_opacity"]), ptr(o["rgb"]),
        ptr(o["clamped"]), ptr(o["tiles_touched"]) if want_tiles else None, P, sh_degree, M, W, H, ptr(gd["means3D"]),
        ptr(gd["scales"]), ptr(gd["rotations"]), ptr(gd["shs"]) if sh_mode else None, ptr(gd["opacities"]), 1.0,
        ptr(V), ptr(PM), ptr(cp), cam.tanfovx, cam.tanfovy, 0, 1, ptr(o["dcolor_ddir"]) if want_ddir else None,
        None, stream()), "gs_preprocess_forward")
    torch.cuda.synchronize()
    return o, gd


def oracle_preprocess(orc, g, cam, sh_mode=True, sh_degree=3):
    n = lambda t: t.numpy()
    return orc.preprocess_fwd(n(g["means3D"]), n(g["scales"]), n(g["rotations"]), n(g["opacities"]),
                              n(g["shs"]) if sh_mode else None, n(cam.world_view_transform),
                              n(cam.full_proj_transform), n(cam.camera_center), cam.image_width, cam.image_height,
                              cam.tanfovx, cam.tanfovy, sh_degree=sh_degree)


def bin_stages(radii, means2D, depths, cl, W, H):
    """Runs the binning stages one by one; returns every intermediate as numpy."""
    P = radii.shape[0]
    gx, gy = grid(W, H)
    T = gx * gy
    tt = torch.empty(P, dtype=torch.int32, device=DEV)
    gn.check(lib.gs_tile_count(P, W, H, ptr(radii), ptr(means2D), ptr(cl), ptr(tt), stream()), "gs_tile_count")
    offs = torch.empty(P, dtype=torch.int32, device=DEV)
    nb = lib.gs_scan_workspace_bytes(P)
    ws = torch.empty(nb, dtype=torch.uint8, device=DEV)
    gn.check(lib.gs_inclusive_sum(P, ptr(tt), ptr(offs), ptr(ws), nb, stream()), "gs_inclusive_sum")
    R = int(np_u32(offs[-1:])[0])
    keys = torch.empty(max(R, 1), dtype=torch.int64, device=DEV)
    vals = torch.empty(max(R, 1), dtype=torch.int32, device=DEV)
    gn.check(lib.gs_duplicate_with_keys(P, W, H, ptr(means2D), ptr(depths), ptr(offs), ptr(radii), ptr(cl), ptr(keys),
                                        ptr(vals), stream()), "gs_duplicate_with_keys")
    keys_u, vals_u = np_u64(keys)[:R].copy(), np_u32(vals)[:R].copy()
    end_bit = 32 + lib.gs_higher_msb(T)
    ks, vs = sort_pairs_u64(keys[:R], vals[:R], end_bit)
    ranges = torch.empty(T, 2, dtype=torch.int32, device=DEV)
    ranges.fill_(-1)
    gn.check(lib.gs_identify_tile_ranges(R, ptr(ks), T, ptr(ranges), stream()), "gs_identify_tile_ranges")
    torch.cuda.synchronize()
    return dict(tiles_touched=np_u32(tt), point_offsets=np_u32(offs), keys_unsorted=keys_u, vals_unsorted=vals_u,
                keys=np_u64(ks), point_list=np_u32(vs), ranges=np_u32(ranges), num_rendered=R, keys_t=ks,
                point_list_t=vs, ranges_t=ranges)


def sort_pairs_u64(keys, vals, end_bit):
    n = keys.shape[0]
    kin, vin = keys.clone(), vals.clone()
    kout, vout = torch.empty_like(kin), torch.empty_like(vin)
    kout.fill_(-1)
    nb = lib.gs_sort_workspace_bytes(n)
    ws = torch.empty(nb, dtype=torch.uint8, device=DEV)
    gn.check(lib.gs_sort_pairs_u64(n, ptr(kin), ptr(kout), ptr(vin), ptr(vout), end_bit, ptr(ws), nb, stream()),
             "gs_sort_pairs_u64")
    if n > 0:
        gn.check(lib.gs_sort_status(ptr(ws), stream()), "gs_sort_status")
    torch.cuda.synchronize()
    return kout, vout


def sort_pairs_u32(keys, vals, end_bit=32):
    n = keys.shape[0]
    kin, vin = keys.clone(), vals.clone()
    kout, vout = torch.empty_like(kin), torch.empty_like(vin)
    nb = lib.gs_sort_workspace_bytes(n)
    ws = torch.empty(nb, dtype=torch.uint8, device=DEV)
    gn.check(lib.gs_sort_pairs_u32(n, ptr(kin), ptr(kout), ptr(vin), ptr(vout), end_bit, ptr(ws), nb, stream()),
             "gs_sort_pairs_u32")
    if n > 0:
        gn.check(lib.gs_sort_status(ptr(ws), stream()), "gs_sort_status")
    torch.cuda.synchronize()
    return kout, vout


def render_fwd(P, W, H, tanx, tany, ranges, point_list, means2D, rgb, all_map, conic_opacity, cl, bg, render_geo=True):
    gx, gy = grid(W, H)
    T = gx * gy
    f = lambda *s: torch.full(s, 55.0, device=DEV)
    i = lambda *s: torch.full(s, 55, dtype=torch.int32, device=DEV)
    o = dict(final_T=f(H, W), n_contrib=i(H, W), n_contrib2loss=i(H, W), color=f(3, H, W),
             out_observe=torch.zeros(P, dtype=torch.int32, device=DEV),
             out_all_map=f(5, H, W) if render_geo else torch.zeros(5, H, W, device=DEV),
             out_plane_depth=f(1, H, W) if render_geo else torch.zeros(1, H, W, device=DEV),
             n_render=i(T), n_consider=i(T), n_contrib_tile=i(T))
    fy = np.float32(H) / (np.float32(2.0) * np.float32(tany))
    fx = np.float32(W) / (np.float32(2.0) * np.float32(tanx))
    gn.check(lib.gs_render_tiles_forward(
        P, W, H, float(fx), float(fy), float(W * 0.5), float(H * 0.5), ptr(ranges), ptr(point_list), ptr(means2D),
        ptr(rgb), ptr(all_map), ptr(conic_opacity), ptr(cl), ptr(bg), int(render_geo), ptr(o["final_T"]),
        ptr(o["n_contrib"]), ptr(o["n_contrib2loss"]), ptr(o["color"]), ptr(o["out_observe"]), ptr(o["out_all_map"]),
        ptr(o["out_plane_depth"]), ptr(o["n_render"]), ptr(o["n_consider"]), ptr(o["n_contrib_tile"]), stream()),
        "gs_render_tiles_forward")
    torch.cuda.synchronize()
    return o


def render_bwd(P, W, H, tanx, tany, bg, ranges, point_list, means2D, conic_opacity, rgb, all_map, all_map_pixels,
               final_T, n_contrib, cl, gpix, gmap, gdepth, emission_sorted, point_offsets, render_geo=True):
    z = lambda *s: torch.full(s, 44.0, device=DEV)  # outputs must be fully overwritten
    o = dict(dL_dmeans2D=z(P, 2), dL_dmeans2D_abs=z(P, 3), dL_dconic_opacity=z(P, 4), dL_dcolors=z(P, 3),
             dL_dall_map=z(P, 5))
    R = int(point_list.shape[0])
    recs = torch.full((max(R, 1), 16), float("nan"), device=DEV)
    gn.check(lib.gs_render_tiles_backward(
        P, W, H, tanx, tany, ptr(bg), ptr(ranges), ptr(point_list), ptr(means2D), ptr(conic_opacity), ptr(rgb),
        ptr(all_map), ptr(all_map_pixels), ptr(final_T), ptr(n_contrib), ptr(cl), ptr(gpix), ptr(gmap), ptr(gdepth),
        int(render_geo), ptr(emission_sorted), ptr(point_offsets), ptr(recs), ptr(o["dL_dmeans2D"]),
        ptr(o["dL_dmeans2D_abs"]), ptr(o["dL_dconic_opacity"]),
        ptr(o["dL_dcolors"]), ptr(o["dL_dall_map"]), stream()), "gs_render_tiles_backward")
    torch.cuda.synchronize()
    return o


def rel_l2(a, b):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    d = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / d) if d > 0 else float(np.linalg.norm(a - b))
