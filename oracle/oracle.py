"""ctypes front end of the CPU oracle (libgs_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke check and the
benchmark's CPU-baseline leg.  The product modules never import this file.

All functions take and return numpy arrays (C-contiguous).  Shapes follow the
reference binding (submodule_cityx/diff-gaussian-rasterization/rasterize_points.cu).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libgs_oracle.so")


def build(force=False):
    """Compile the oracle with the Makefile beside this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-B", "-C", _HERE, "libgs_oracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.oracle_higher_msb.restype = C.c_uint32
        _lib.oracle_higher_msb.argtypes = [C.c_uint32]
        _lib.oracle_morton.restype = C.c_uint32
        _lib.oracle_num_threads.restype = C.c_int
    return _lib


def _p(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a):
    return np.ascontiguousarray(np.asarray(a).astype(np.uint8))


def num_threads():
    return lib().oracle_num_threads()


def set_num_threads(n):
    lib().oracle_set_num_threads(C.c_int(n))


def expf(x):
    x = _f32(x).ravel()
    y = np.empty_like(x)
    lib().oracle_expf(C.c_int(x.size), _p(x), _p(y))
    return y


def higher_msb(n):
    return int(lib().oracle_higher_msb(C.c_uint32(n)))


def tile_grid(W, H):
    return (W + 15) // 16, (H + 15) // 16


def mark_visible(means, V, PM):
    means, V, PM = _f32(means), _f32(V), _f32(PM)
    P = means.shape[0]
    out = np.zeros(P, np.uint8)
    lib().oracle_mark_visible(C.c_int(P), _p(means), _p(V), _p(PM), _p(out))
    return out.astype(bool)


def preprocess_fwd(means, scales, rots, opac, shs, V, PM, campos, W, H, tanx, tany, sh_degree=3, mod=1.0):
    """shs is None / (P,3) (reference-compatible: colour untouched) or (P,M,3) (SH mode)."""
    means, scales, rots, opac = _f32(means), _f32(scales), _f32(rots), _f32(opac)
    V, PM, campos = _f32(V), _f32(PM), _f32(campos)
    P = means.shape[0]
    sh_mode = shs is not None and np.ndim(shs) == 3
    M = shs.shape[1] if sh_mode else 0
    shs_c = _f32(shs) if sh_mode else None
    o = dict(
        radii=np.zeros(P, np.int32),
        means2D=np.zeros((P, 2), np.float32),
        depths=np.zeros(P, np.float32),
        cov3D=np.zeros((P, 6), np.float32),
        conic_opacity=np.zeros((P, 4), np.float32),
        rgb=np.zeros((P, 3), np.float32),
        clamped=np.zeros((P, 3), np.uint8),
        tiles_touched=np.zeros(P, np.uint32),
    )
    lib().oracle_preprocess_fwd(
        C.c_int(P), C.c_int(sh_degree), C.c_int(M), _p(means), _p(scales), C.c_float(mod), _p(rots), _p(opac),
        _p(shs_c), _p(V), _p(PM), _p(campos), C.c_int(W), C.c_int(H), C.c_float(tanx), C.c_float(tany),
        _p(o["radii"]), _p(o["means2D"]), _p(o["depths"]), _p(o["cov3D"]), _p(o["conic_opacity"]), _p(o["rgb"]),
        _p(o["clamped"]), _p(o["tiles_touched"]))
    return o


def visible_filter(means, scales, rots, cov_pre, V, PM, W, H, tanx, tany, mod=1.0):
    means, V, PM = _f32(means), _f32(V), _f32(PM)
    P = means.shape[0]
    scales = _f32(scales) if scales is not None else None
    rots = _f32(rots) if rots is not None else None
    cov_pre = _f32(cov_pre) if cov_pre is not None else None
    radii = np.zeros(P, np.int32)
    lib().oracle_visible_filter(C.c_int(P), _p(means), _p(scales), C.c_float(mod), _p(rots), _p(cov_pre), _p(V),
                                _p(PM), C.c_int(W), C.c_int(H), C.c_float(tanx), C.c_float(tany), _p(radii))
    return radii


def tiles_touched(radii, means2D, compute_locally, W, H):
    radii = np.ascontiguousarray(radii, np.int32)
    means2D = _f32(means2D)
    cl = _u8(compute_locally).ravel()
    P = radii.shape[0]
    out = np.zeros(P, np.uint32)
    lib().oracle_tiles_touched(C.c_int(P), C.c_int(W), C.c_int(H), _p(radii), _p(means2D), _p(cl), _p(out))
    return out


def inclusive_sum(x):
    x = np.ascontiguousarray(x, np.uint32)
    out = np.empty_like(x)
    lib().oracle_inclusive_sum(C.c_int(x.size), _p(x), _p(out))
    return out


def duplicate_with_keys(means2D, depths, offsets, radii, compute_locally, W, H):
    means2D, depths = _f32(means2D), _f32(depths)
    offsets = np.ascontiguousarray(offsets, np.uint32)
    radii = np.ascontiguousarray(radii, np.int32)
    cl = _u8(compute_locally).ravel()
    P = radii.shape[0]
    R = int(offsets[-1]) if P else 0
    keys = np.zeros(R, np.uint64)
    vals = np.zeros(R, np.uint32)
    lib().oracle_duplicate_with_keys(C.c_int(P), C.c_int(W), C.c_int(H), _p(means2D), _p(depths), _p(offsets),
                                     _p(radii), _p(cl), _p(keys), _p(vals))
    return keys, vals


def sort_pairs(keys, vals, end_bit=64):
    keys = np.ascontiguousarray(keys, np.uint64)
    vals = np.ascontiguousarray(vals, np.uint32)
    ko, vo = np.empty_like(keys), np.empty_like(vals)
    lib().oracle_sort_pairs(C.c_int64(keys.size), _p(keys), _p(vals), _p(ko), _p(vo), C.c_int(end_bit))
    return ko, vo


def sort_pairs_u32(keys, vals):
    keys = np.ascontiguousarray(keys, np.uint32)
    vals = np.ascontiguousarray(vals, np.uint32)
    ko, vo = np.empty_like(keys), np.empty_like(vals)
    lib().oracle_sort_pairs_u32(C.c_int64(keys.size), _p(keys), _p(vals), _p(ko), _p(vo))
    return ko, vo


def tile_ranges(keys_sorted, T):
    keys_sorted = np.ascontiguousarray(keys_sorted, np.uint64)
    ranges = np.zeros((T, 2), np.uint32)
    lib().oracle_tile_ranges(C.c_int64(keys_sorted.size), _p(keys_sorted), C.c_int(T), _p(ranges))
    return ranges


def bin_and_sort(radii, means2D, depths, compute_locally, W, H):
    """updateTileTouched -> InclusiveSum -> duplicateWithKeys -> SortPairs -> identifyTileRanges
    (renderForward, cuda_rasterizer/rasterizer_impl.cu:633-697)."""
    gx, gy = tile_grid(W, H)
    tt = tiles_touched(radii, means2D, compute_locally, W, H)
    offs = inclusive_sum(tt)
    keys, vals = duplicate_with_keys(means2D, depths, offs, radii, compute_locally, W, H)
    bit = higher_msb(gx * gy)
    ks, vs = sort_pairs(keys, vals, 32 + bit)
    ranges = tile_ranges(ks, gx * gy)
    # the permutation the stable sort applied: sorted position -> index in emission order
    mask = np.uint64((1 << (32 + bit)) - 1)
    emission_sorted = np.argsort(keys & mask, kind="stable").astype(np.uint32)
    return dict(tiles_touched=tt, point_offsets=offs, keys_unsorted=keys, vals_unsorted=vals, keys=ks,
                point_list=vs, ranges=ranges, num_rendered=int(keys.size), emission_sorted=emission_sorted)


def render_fwd(ranges, point_list, means2D, rgb, all_map, conic_opacity, compute_locally, bg, W, H, tanx, tany,
               render_geo=True):
    ranges = np.ascontiguousarray(ranges, np.uint32)
    point_list = np.ascontiguousarray(point_list, np.uint32)
    means2D, rgb, all_map, conic_opacity, bg = _f32(means2D), _f32(rgb), _f32(all_map), _f32(conic_opacity), _f32(bg)
    cl = _u8(compute_locally).ravel()
    P = means2D.shape[0]
    o = dict(
        final_T=np.zeros((H, W), np.float32),
        n_contrib=np.zeros((H, W), np.uint32),
        n_contrib2loss=np.zeros((H, W), np.uint32),
        color=np.zeros((3, H, W), np.float32),
        out_observe=np.zeros(P, np.int32),
        out_all_map=np.zeros((5, H, W), np.float32),
        out_plane_depth=np.zeros((1, H, W), np.float32),
    )
    lib().oracle_render_fwd(C.c_int(W), C.c_int(H), C.c_float(tanx), C.c_float(tany), _p(ranges), _p(point_list),
                            _p(means2D), _p(rgb), _p(all_map), _p(conic_opacity), _p(cl), _p(bg),
                            C.c_int(int(render_geo)), _p(o["final_T"]), _p(o["n_contrib"]), _p(o["n_contrib2loss"]),
                            _p(o["color"]), _p(o["out_observe"]), _p(o["out_all_map"]), _p(o["out_plane_depth"]))
    gx, gy = tile_grid(W, H)
    T = gx * gy
    o["n_render"] = np.zeros(T, np.int32)
    o["n_consider"] = np.zeros(T, np.int32)
    o["n_contrib_tile"] = np.zeros(T, np.int32)
    lib().oracle_tile_stats(C.c_int(W), C.c_int(H), _p(ranges), _p(o["n_contrib"]), _p(o["n_contrib2loss"]), _p(cl),
                            _p(o["n_render"]), _p(o["n_consider"]), _p(o["n_contrib_tile"]))
    return o


def max_weight_depth(ranges, point_list, means2D, conic_opacity, depths, compute_locally, W, H):
    """Per pixel the depth of the Gaussian that blends with the largest weight (no reference counterpart; defined
    by oracle_max_weight_depth).  (1, H, W); pixels of tiles that are not computed locally stay 0."""
    ranges = np.ascontiguousarray(ranges, np.uint32)
    point_list = np.ascontiguousarray(point_list, np.uint32)
    means2D, conic_opacity, depths = _f32(means2D), _f32(conic_opacity), _f32(depths)
    cl = _u8(compute_locally).ravel()
    out = np.zeros((1, H, W), np.float32)
    lib().oracle_max_weight_depth(C.c_int(W), C.c_int(H), _p(ranges), _p(point_list), _p(means2D), _p(conic_opacity),
                                  _p(depths), _p(cl), _p(out))
    return out


def render_bwd(ranges, point_list, means2D, conic_opacity, rgb, all_map, all_map_pixels, final_T, n_contrib,
               compute_locally, bg, dL_dpix, dL_dout_all_map, dL_dout_plane_depth, W, H, tanx, tany, render_geo=True):
    ranges = np.ascontiguousarray(ranges, np.uint32)
    point_list = np.ascontiguousarray(point_list, np.uint32)
    means2D, rgb, all_map, conic_opacity, bg = _f32(means2D), _f32(rgb), _f32(all_map), _f32(conic_opacity), _f32(bg)
    all_map_pixels, final_T = _f32(all_map_pixels), _f32(final_T)
    n_contrib = np.ascontiguousarray(n_contrib, np.uint32)
    dL_dpix, dL_dout_all_map, dL_dout_plane_depth = _f32(dL_dpix), _f32(dL_dout_all_map), _f32(dL_dout_plane_depth)
    cl = _u8(compute_locally).ravel()
    P = means2D.shape[0]
    o = dict(
        dL_dmeans2D=np.zeros((P, 3), np.float32),
        dL_dmeans2D_abs=np.zeros((P, 3), np.float32),
        dL_dconic=np.zeros((P, 4), np.float32),
        dL_dopacity=np.zeros((P, 1), np.float32),
        dL_dcolors=np.zeros((P, 3), np.float32),
        dL_dall_map=np.zeros((P, 5), np.float32),
    )
    lib().oracle_render_bwd(C.c_int(P), C.c_int(W), C.c_int(H), C.c_float(tanx), C.c_float(tany), _p(bg), _p(ranges),
                            _p(point_list), _p(means2D), _p(conic_opacity), _p(rgb), _p(all_map), _p(all_map_pixels),
                            _p(final_T), _p(n_contrib), _p(cl), _p(dL_dpix), _p(dL_dout_all_map),
                            _p(dL_dout_plane_depth), C.c_int(int(render_geo)), _p(o["dL_dmeans2D"]),
                            _p(o["dL_dmeans2D_abs"]), _p(o["dL_dconic"]), _p(o["dL_dopacity"]), _p(o["dL_dcolors"]),
                            _p(o["dL_dall_map"]))
    # packed form returned by the binding (rasterize_points.cu:428-440): [conic.x, conic.y, conic.w, opacity]
    d = o["dL_dconic"]
    o["dL_dconic_opacity"] = np.stack([d[:, 0], d[:, 1], d[:, 3], o["dL_dopacity"][:, 0]], axis=1)
    return o


def preprocess_bwd(means, radii, shs, clamped, scales, rots, cov3D, V, PM, campos, W, H, tanx, tany, dL_dmeans2D,
                   dL_dconic_opacity, dL_dcolor, sh_degree=3, mod=1.0):
    """dL_dmeans2D (P,2) or (P,3); dL_dconic_opacity (P,4) packed [x, y, w, opacity]
    (rasterize_points.cu:181-194).  Returns the five gradients of the binding."""
    means, scales, rots, cov3D = _f32(means), _f32(scales), _f32(rots), _f32(cov3D)
    V, PM, campos = _f32(V), _f32(PM), _f32(campos)
    radii = np.ascontiguousarray(radii, np.int32)
    P = means.shape[0]
    sh_mode = shs is not None and np.ndim(shs) == 3
    M = shs.shape[1] if sh_mode else 0
    shs_c = _f32(shs) if sh_mode else None
    g2 = np.zeros((P, 3), np.float32)
    g2[:, :2] = _f32(dL_dmeans2D)[:, :2]
    gco = _f32(dL_dconic_opacity)
    gconic = np.zeros((P, 4), np.float32)
    gconic[:, 0], gconic[:, 1], gconic[:, 3] = gco[:, 0], gco[:, 1], gco[:, 2]
    gcol = _f32(dL_dcolor) if dL_dcolor is not None else np.zeros((P, 3), np.float32)
    cl = _u8(clamped) if clamped is not None else np.zeros((P, 3), np.uint8)
    o = dict(
        dL_dmeans3D=np.zeros((P, 3), np.float32),
        dL_dcov3D=np.zeros((P, 6), np.float32),
        dL_dscales=np.zeros((P, 3), np.float32),
        dL_drotations=np.zeros((P, 4), np.float32),
        dL_dsh=np.zeros((P, M, 3) if sh_mode else (P, 3), np.float32),
        dL_dopacity=gco[:, 3:4].copy(),
    )
    lib().oracle_preprocess_bwd(C.c_int(P), C.c_int(sh_degree), C.c_int(M), _p(means), _p(radii), _p(shs_c), _p(cl),
                                _p(scales), _p(rots), C.c_float(mod), _p(cov3D), _p(V), _p(PM), C.c_int(W), C.c_int(H),
                                C.c_float(tanx), C.c_float(tany), _p(campos), _p(g2), _p(gconic), _p(gcol),
                                _p(o["dL_dmeans3D"]), _p(o["dL_dcov3D"]), _p(o["dL_dsh"]) if sh_mode else None,
                                _p(o["dL_dscales"]), _p(o["dL_drotations"]))
    return o


def all_map_fwd(means3D, scales, rotations, viewmatrix, campos):
    """gaussian_renderer/__init__.py:1501-1518."""
    means3D, scales, rotations = _f32(means3D), _f32(scales), _f32(rotations)
    V, cp = _f32(viewmatrix).reshape(16), _f32(campos).reshape(3)
    P = means3D.shape[0]
    out = np.zeros((P, 5), np.float32)
    lib().oracle_all_map_fwd(C.c_int(P), _p(means3D), _p(scales), _p(rotations), _p(V), _p(cp), _p(out))
    return out


def all_map_bwd(means3D, scales, rotations, viewmatrix, campos, grad_out):
    means3D, scales, rotations, grad_out = _f32(means3D), _f32(scales), _f32(rotations), _f32(grad_out)
    V, cp = _f32(viewmatrix).reshape(16), _f32(campos).reshape(3)
    P = means3D.shape[0]
    dm, dq = np.zeros((P, 3), np.float32), np.zeros((P, 4), np.float32)
    lib().oracle_all_map_bwd(C.c_int(P), _p(means3D), _p(scales), _p(rotations), _p(V), _p(cp), _p(grad_out), _p(dm),
                             _p(dq))
    return dm, dq


def ssim_window():
    """The 11 normalised 1-D weights of create_window (utils/loss_utils.py:27-43) as float32: exp in Python
    floats, stored as float32, divided by their float32 sum."""
    import math
    g = np.array([math.exp(-((x - 11 // 2) ** 2) / float(2 * 1.5 ** 2)) for x in range(11)], np.float32)
    return (g / g.sum(dtype=np.float32)).astype(np.float32)


def ssim_l1_fwd(img1, img2, mask=None):
    """pixelwise_l1_with_mask, pixelwise_ssim_with_mask (utils/loss_utils.py:88-132): (l1_map, ssim_map)."""
    img1, img2 = _f32(img1), _f32(img2)
    Cn, H, W = img1.shape
    m = None if mask is None else _u8(mask).reshape(H, W)
    l1, ss = np.zeros_like(img1), np.zeros_like(img1)
    lib().oracle_ssim_l1_fwd(C.c_int(Cn), C.c_int(H), C.c_int(W), _p(img1), _p(img2), _p(m) if m is not None else None,
                             _p(ssim_window()), _p(l1), _p(ss))
    return l1, ss


def ssim_l1_bwd(img1, img2, mask, g_l1, g_ssim):
    img1, img2, g_l1, g_ssim = _f32(img1), _f32(img2), _f32(g_l1), _f32(g_ssim)
    Cn, H, W = img1.shape
    m = None if mask is None else _u8(mask).reshape(H, W)
    d = np.zeros_like(img1)
    lib().oracle_ssim_l1_bwd(C.c_int(Cn), C.c_int(H), C.c_int(W), _p(img1), _p(img2),
                             _p(m) if m is not None else None, _p(ssim_window()), _p(g_l1), _p(g_ssim), _p(d))
    return d


def training_stats(opacity_accum, anchor_demon, grad_accum, denom, k, grad, opacity, update_filter,
                   offset_selection_mask, anchor_visible_mask):
    """GaussianModel.training_statis (scene/gaussian_model.py:1181-1205) with the mask gathers and scatters
    written out as ranks: returns the four updated accumulators (flattened float32)."""
    oa, ad = _f32(opacity_accum).ravel().copy(), _f32(anchor_demon).ravel().copy()
    ga, dn = _f32(grad_accum).ravel().copy(), _f32(denom).ravel().copy()
    vis = np.asarray(anchor_visible_mask).astype(bool).ravel()
    sel = np.asarray(offset_selection_mask).astype(bool).ravel()
    flt = np.asarray(update_filter).astype(bool).ravel()
    op, g = _f32(opacity).ravel(), _f32(grad)
    rank_vis = np.cumsum(vis) - vis      # exclusive count of visible anchors
    rank_sel = np.cumsum(sel) - sel      # exclusive count of selected candidates
    for a in np.nonzero(vis)[0]:
        first = int(rank_vis[a]) * k
        s = np.float32(0)
        for j in range(k):
            o = op[first + j]
            s = np.float32(s + (np.float32(0) if o < 0 else o))    # :1183-1187
        oa[a] += s
        ad[a] += np.float32(1)                                       # :1190
        for j in range(k):
            i = first + j
            if sel[i]:                                               # combined_mask[anchor_visible] = offset_selection
                r = int(rank_sel[i])
                if flt[r]:                                           # combined_mask[temp_mask] = update_filter
                    ga[a * k + j] += np.sqrt(g[r, 0] * g[r, 0] + g[r, 1] * g[r, 1])   # :1203-1204
                    dn[a * k + j] += np.float32(1)                                     # :1205
    return oa, ad, ga, dn


def adam_step(param, grad, exp_avg, exp_avg_sq, lr, step, beta1=0.9, beta2=0.999, eps=1e-15, grad_scale=1.0):
    """One torch.optim.Adam update (torch 2.0.0 rule, no weight decay / amsgrad; the optimizer of
    scene/gaussian_model.py:574) in float32 numpy, returning new (param, exp_avg, exp_avg_sq).  Bias corrections
    are Python floats, as in torch/optim/adam.py."""
    f = np.float32
    p, g, m, v = _f32(param), _f32(grad) * f(grad_scale), _f32(exp_avg), _f32(exp_avg_sq)
    m = m * f(beta1) + f(1.0 - beta1) * g
    v = v * f(beta2) + (f(1.0 - beta2) * g) * g
    bc1 = 1.0 - beta1 ** step
    bc2 = 1.0 - beta2 ** step
    neg_step = f(-(lr / bc1))
    denom = np.sqrt(v) / f(np.sqrt(bc2)) + f(eps)
    p = p + (neg_step * m) / denom
    return p.astype(np.float32), m.astype(np.float32), v.astype(np.float32)


def knn_dist2(points):
    points = _f32(points)
    P = points.shape[0]
    out = np.zeros(P, np.float32)
    lib().oracle_knn_dist2(C.c_int(P), _p(points), _p(out))
    return out


def morton(p, mn, mx):
    p, mn, mx = _f32(p), _f32(mn), _f32(mx)
    return int(lib().oracle_morton(_p(p), _p(mn), _p(mx)))


def _mlp_args(mlps, input_flags=0):
    """mlps: three (W1 (32, 35 + extra inputs), b1 (32), W2 (out,32), b2 (out)) tuples in the order opacity, color,
    cov; extra inputs of MLP m: the distance if bit m of input_flags is set, the level if bit 3 is."""
    flat = []
    for m, (W1, b1, W2, b2) in enumerate(mlps):
        assert W1.shape == (32, 35 + ((input_flags >> m) & 1) + ((input_flags >> 3) & 1)), W1.shape
        flat += [_f32(W1), _f32(b1), _f32(W2), _f32(b2)]
    return flat


def neural_gaussians_fwd(anchor, feat, offsets, scaling, campos, mlps, prog=None, level=None, input_flags=0):
    """generate_neural_gaussians (gaussian_renderer/__init__.py:789-899), default configuration, on the anchors
    already selected by visible_mask; prog (N), if given, is the per-anchor factor of dist2level 'progressive'
    (:844-848); input_flags / level: the MLPs' optional distance and level inputs (add_opacity_dist = 1,
    add_color_dist = 2, add_cov_dist = 4, add_level = 8; :824-877).
    Returns (xyz, color, opacity, scaling, rot, neural_opacity, mask)."""
    anchor, feat, offsets, scaling = _f32(anchor), _f32(feat), _f32(offsets), _f32(scaling)
    cp = _f32(campos).reshape(3)
    N, k = anchor.shape[0], offsets.shape[1]
    w = _mlp_args(mlps, input_flags)
    lv = None if level is None else _f32(level).reshape(N)
    assert lv is not None or not (input_flags & 8)
    nop, mask = np.zeros((N * k, 1), np.float32), np.zeros(N * k, np.uint8)
    col, sr = np.zeros((N * k, 3), np.float32), np.zeros((N * k, 7), np.float32)
    pg = None if prog is None else _f32(prog).reshape(N)
    lib().oracle_neural_mlp_fwd(C.c_int(N), C.c_int(k), _p(anchor), _p(feat), _p(cp), *[_p(x) for x in w],
                                None if pg is None else _p(pg), None if lv is None else _p(lv),
                                C.c_int(input_flags), _p(nop), _p(mask), _p(col), _p(sr))
    S = int(mask.sum())
    xyz, c, op = np.zeros((S, 3), np.float32), np.zeros((S, 3), np.float32), np.zeros((S, 1), np.float32)
    sc, rot = np.zeros((S, 3), np.float32), np.zeros((S, 4), np.float32)
    lib().oracle_neural_compact.restype = C.c_int
    got = lib().oracle_neural_compact(C.c_int(N), C.c_int(k), _p(anchor), _p(offsets), _p(scaling), _p(nop), _p(mask),
                                      _p(col), _p(sr), _p(xyz), _p(c), _p(op), _p(sc), _p(rot))
    assert got == S
    return xyz, c, op, sc, rot, nop, mask.astype(bool)


def neural_gaussians_bwd(anchor, feat, offsets, scaling, campos, mlps, g_xyz, g_color, g_opacity, g_scaling, g_rot,
                         prog=None, level=None, input_flags=0):
    """Gradients of neural_gaussians_fwd's five compacted outputs: (d_anchor, d_feat, d_offsets, d_scaling,
    [12 weight gradients in the order of mlps])."""
    anchor, feat, offsets, scaling = _f32(anchor), _f32(feat), _f32(offsets), _f32(scaling)
    cp = _f32(campos).reshape(3)
    N, k = anchor.shape[0], offsets.shape[1]
    w = _mlp_args(mlps, input_flags)
    lv = None if level is None else _f32(level).reshape(N)
    gs = [_f32(g_xyz), _f32(g_color), _f32(g_opacity), _f32(g_scaling), _f32(g_rot)]
    da, df = np.zeros((N, 3), np.float32), np.zeros((N, 32), np.float32)
    do, ds = np.zeros((N, k, 3), np.float32), np.zeros((N, 6), np.float32)
    dw = [np.zeros_like(x) for x in w]
    pg = None if prog is None else _f32(prog).reshape(N)
    lib().oracle_neural_bwd(C.c_int(N), C.c_int(k), _p(anchor), _p(feat), _p(offsets), _p(scaling), _p(cp),
                            *[_p(x) for x in w], None if pg is None else _p(pg), None if lv is None else _p(lv),
                            C.c_int(input_flags), *[_p(x) for x in gs], _p(da), _p(df), _p(do), _p(ds),
                            *[_p(x) for x in dw])
    return da, df, do, ds, dw
