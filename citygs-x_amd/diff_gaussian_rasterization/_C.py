"""Drop-in for the reference's compiled extension module
(submodule_cityx/diff-gaussian-rasterization/ext.cpp:16-35): same function
names, argument order and return tuples, implemented on libgsrast.so through
ctypes.  torch is used for device memory and the current stream only.
"""
import ctypes as C
import os

import numpy as np
import torch

import gsrast_native as _n

_lib = _n.lib
BLOCK_X, BLOCK_Y, ONE_DIM_BLOCK_SIZE = 16, 16, 256
NUM_CHANNELS, NUM_ALL_MAP = 3, 5

# When True, render forward/backward are timed with events and the call blocks
# until the kernels finish, like the reference (rasterizer_impl.cu:754-755,
# :924-926).  When False the stats_collector entries are written as 0.0 and no
# host synchronisation is added.  cuda_args["zhx_time"] == "True" also enables it.
TIME_RENDER = False


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream(device):
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _f32c(t, name):
    if t.dtype != torch.float32:
        raise TypeError(f"{name} must be float32, got {t.dtype}")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a GPU tensor: this rasterizer has no CPU path")
    return t.contiguous()


def _want_timing(cuda_args):
    if TIME_RENDER:
        return True
    try:
        return cuda_args is not None and str(cuda_args.get("zhx_time", "False")) == "True"
    except AttributeError:
        return False


def _record_time(cuda_args, key, value):
    if cuda_args is None:
        return
    sc = cuda_args.get("stats_collector") if hasattr(cuda_args, "get") else None
    if sc is not None:
        sc[key] = float(value)


def get_block_XY():
    """rasterize_points.cu:858-861."""
    bx, by, od = C.c_int(), C.c_int(), C.c_int()
    _n.check(_lib.gs_get_block_xy(C.byref(bx), C.byref(by), C.byref(od)), "get_block_XY")
    return bx.value, by.value, od.value


def mark_visible(means3D, viewmatrix, projmatrix):
    """rasterize_points.cu:39-58."""
    means3D = _f32c(means3D, "means3D")
    P = means3D.shape[0]
    present = torch.zeros(P, dtype=torch.bool, device=means3D.device)
    if P != 0:
        vm, pm = _f32c(viewmatrix, "viewmatrix"), _f32c(projmatrix, "projmatrix")
        with torch.cuda.device(means3D.device):
            _n.check(_lib.gs_mark_visible(P, _ptr(means3D), _ptr(vm), _ptr(pm), _ptr(present), _stream(means3D.device)),
                     "mark_visible")
    return present


def preprocess_gaussians(means3D, scales, rotations, sh, opacity, scale_modifier, viewmatrix, projmatrix, tan_fovx,
                         tan_fovy, image_height, image_width, degree, campos, prefiltered, debug, args):
    """rasterize_points.cu:63-143.  A 3-D `sh` (P,M,3) switches the SH colour
    step on; any other shape keeps the reference behaviour (rgb stays zero)."""
    return preprocess_gaussians_ex(means3D, scales, rotations, sh, opacity, scale_modifier, viewmatrix, projmatrix,
                                   tan_fovx, tan_fovy, image_height, image_width, degree, campos, prefiltered, debug,
                                   args)[0]


def preprocess_gaussians_ex(means3D, scales, rotations, sh, opacity, scale_modifier, viewmatrix, projmatrix, tan_fovx,
                            tan_fovy, image_height, image_width, degree, campos, prefiltered, debug, args,
                            want_direction_derivative=False, want_cov3D=True, blend_records=None):
    """preprocess_gaussians plus what the reference's tuple has no slot for: returns (tuple, dcolor_ddir).  With
    want_direction_derivative (and SH colours) dcolor_ddir is the (P,3,3) derivative of every surviving Gaussian's
    colour with respect to the unit view direction; handed to preprocess_gaussians_backward it replaces the
    coefficients there (same gradients, and the backward pass does not read the 192-byte rows).  Otherwise None.
    want_cov3D=False leaves the cov3D slot of the tuple None: preprocess_gaussians_backward, given None, forms the
    covariances again from scales and rotations (the same bits), and neither pass moves the 24 bytes per Gaussian.
    blend_records: an optional (P,16) float32 tensor that receives the blend kernels' operand records of the
    surviving Gaussians, geometry channels included (those build_all_map gives for the same means3D, scales,
    rotations, viewmatrix and campos); see render_gaussians_ex."""
    if means3D.ndimension() != 2 or means3D.size(1) != 3:
        raise RuntimeError("means3D must have dimensions (num_points, 3)")
    means3D = _f32c(means3D, "means3D")
    dev = means3D.device
    P = means3D.shape[0]
    f32 = dict(dtype=torch.float32, device=dev)
    if P == 0:
        return ((0, torch.zeros(0, 2, **f32), torch.zeros(0, **f32), torch.zeros(0, dtype=torch.int32, device=dev),
                 torch.zeros(0, 6, **f32), torch.zeros(0, 4, **f32), torch.zeros(0, 3, **f32),
                 torch.zeros(0, 3, dtype=torch.bool, device=dev)), None)
    means2D = torch.empty(P, 2, **f32)
    depths = torch.empty(P, **f32)
    radii = torch.empty(P, dtype=torch.int32, device=dev)
    cov3D = torch.empty(P, 6, **f32) if want_cov3D else None
    conic_opacity = torch.empty(P, 4, **f32)
    rgb = torch.empty(P, 3, **f32)
    clamped = torch.empty(P, 3, dtype=torch.bool, device=dev)
    scales, rotations, opacity = _f32c(scales, "scales"), _f32c(rotations, "rotations"), _f32c(opacity, "opacity")
    vm, pm, cp = _f32c(viewmatrix, "viewmatrix"), _f32c(projmatrix, "projmatrix"), _f32c(campos, "campos")
    sh_mode = sh is not None and sh.dim() == 3 and sh.shape[0] == P
    M = sh.shape[1] if sh_mode else 0
    shc = _f32c(sh, "sh") if sh_mode else None
    ddir = torch.empty(P, 3, 3, **f32) if (sh_mode and want_direction_derivative) else None
    with torch.cuda.device(dev):
        _n.check(_lib.gs_preprocess_forward(
            _ptr(means2D), _ptr(depths), _ptr(radii), _ptr(cov3D), _ptr(conic_opacity), _ptr(rgb), _ptr(clamped), None,
            P, int(degree), M, int(image_width), int(image_height), _ptr(means3D), _ptr(scales), _ptr(rotations),
            _ptr(shc), _ptr(opacity), float(scale_modifier), _ptr(vm), _ptr(pm), _ptr(cp), float(tan_fovx),
            float(tan_fovy), int(bool(prefiltered)), int(bool(debug)), _ptr(ddir), _ptr(blend_records),
            _stream(dev)),
            "preprocess_gaussians")
    return (0, means2D, depths, radii, cov3D, conic_opacity, rgb, clamped), ddir


def preprocess_gaussians_backward(radii, cov3D, clamped, means3D, scales, rotations, sh, scale_modifier, viewmatrix,
                                  projmatrix, tan_fovx, tan_fovy, image_height, image_width, degree, campos,
                                  dL_dmeans2D, dL_dconic_opacity, dL_dcolors, R, debug, args, dcolor_ddir=None):
    """rasterize_points.cu:146-234.  dL_dmeans2D may be (P,2) or (P,3).  dcolor_ddir: what
    preprocess_gaussians_ex returned for the same inputs, or None."""
    means3D = _f32c(means3D, "means3D")
    dev = means3D.device
    P = means3D.shape[0]
    f32 = dict(dtype=torch.float32, device=dev)
    sh_mode = sh is not None and sh.dim() == 3 and sh.shape[0] == P
    M = sh.shape[1] if sh_mode else 0
    dL_dsh = torch.empty(P, M, 3, **f32) if sh_mode else torch.zeros(P, 3, **f32)
    if P == 0:
        return (torch.zeros(0, 3, **f32), torch.zeros(0, 3, **f32), torch.zeros(0, 4, **f32), dL_dsh,
                torch.zeros(0, 1, **f32))
    dL_dmeans3D = torch.empty(P, 3, **f32)
    dL_dscales = torch.empty(P, 3, **f32)
    dL_drotations = torch.empty(P, 4, **f32)
    dL_dopacity = torch.empty(P, 1, **f32)
    g2 = _f32c(dL_dmeans2D, "dL_dmeans2D")
    gco = _f32c(dL_dconic_opacity, "dL_dconic_opacity")
    gcol = _f32c(dL_dcolors, "dL_dcolors") if (sh_mode and dL_dcolors is not None) else None
    if sh_mode and gcol is None:
        gcol = torch.zeros(P, 3, **f32)
    scales, rotations = _f32c(scales, "scales"), _f32c(rotations, "rotations")
    vm, pm, cp = _f32c(viewmatrix, "viewmatrix"), _f32c(projmatrix, "projmatrix"), _f32c(campos, "campos")
    shc = _f32c(sh, "sh") if sh_mode else None
    with torch.cuda.device(dev):
        _n.check(_lib.gs_preprocess_backward(
            _ptr(radii.contiguous()), _ptr(cov3D.contiguous() if cov3D is not None else None),
            _ptr(clamped.contiguous()), P, int(degree), M,
            int(image_width), int(image_height), _ptr(means3D), _ptr(scales), _ptr(rotations), _ptr(shc),
            float(scale_modifier), _ptr(vm), _ptr(pm), _ptr(cp), float(tan_fovx), float(tan_fovy), _ptr(g2),
            int(g2.shape[1]), _ptr(gco), _ptr(gcol), _ptr(dL_dmeans3D), None, _ptr(dL_dscales), _ptr(dL_drotations),
            _ptr(dL_dsh) if sh_mode else None, _ptr(dL_dopacity), int(bool(debug)),
            _ptr(dcolor_ddir) if (sh_mode and dcolor_ddir is not None) else None, _stream(dev)),
            "preprocess_gaussians_backward")
    return dL_dmeans3D, dL_dscales, dL_drotations, dL_dsh, dL_dopacity


class _GrowBuffer:
    """Byte tensor grown on demand by the native side (resizeFunctional,
    rasterize_points.cu:31-37)."""

    def __init__(self, device):
        self.device = device
        self.tensor = torch.empty(0, dtype=torch.uint8, device=device)
        self.callback = _n.RESIZE_FN(self._resize)

    def _resize(self, nbytes, _user):
        if self.tensor.numel() < nbytes:
            self.tensor = torch.empty(int(nbytes), dtype=torch.uint8, device=self.device)
        return self.tensor.data_ptr()

    def release(self):
        # drop the callback so this object does not keep the tensor alive through a reference cycle
        self.callback = None
        return self.tensor


def render_gaussians(background, image_height, image_width, means2D, depths, radii, conic_opacity, rgb,
                     compute_locally, viewmatrix, campos, tan_fovx, tan_fovy, all_map, render_geo, debug, args):
    """rasterize_points.cu:276-364.  Two additions: with args["max_weight_depth"] set, the per-pixel depth of the
    Gaussian that blends with the largest weight (1, H, W) is left in args["stats_collector"]["max_weight_depth"];
    args["tile_sort_limits"] = (small_limit, block_records) chooses, for this call, the way the per-tile
    lists are built (the longest list sorted in registers, 0 = one radix sort over all keys; the records the
    per-tile radix sort holds at once; all ways give the same lists).  The returned tuple is the reference's either way."""
    return render_gaussians_ex(background, image_height, image_width, means2D, depths, radii, conic_opacity, rgb,
                               compute_locally, viewmatrix, campos, tan_fovx, tan_fovy, all_map, render_geo, debug,
                               args)[0]


def _want_tile_log(args):
    """cuda_rasterizer/rasterizer_impl.cu:764: in training, with zhx_debug, on the first iteration of every
    log interval."""
    if not isinstance(args, dict):
        return False
    try:
        return (str(args.get("mode", "")) == "train" and str(args.get("zhx_debug", "False")) == "True"
                and int(args.get("iteration", 0)) % int(args.get("log_interval", 0) or 1) == 1)
    except (TypeError, ValueError):
        return False


def _write_tile_log(args, H, W, n_render, n_consider, n_contrib):
    """The reference's per-tile debug log (cuda_rasterizer/rasterizer_impl.cu:764-842, file name and line prefix
    from save_log_in_file, :290-298): for every tile with a non-empty list its range, the list length and the
    per-pixel averages of the two contributor counts, then one line of totals.  The per-tile sums the reference
    forms on the host from the per-pixel images are the three per-tile outputs of the forward call."""
    gx, gy = (W + BLOCK_X - 1) // BLOCK_X, (H + BLOCK_Y - 1) // BLOCK_Y
    nr = n_render.cpu().numpy().astype(np.int64)
    nc = n_consider.cpu().numpy().astype(np.int64)
    n2 = n_contrib.cpu().numpy().astype(np.int64)
    ends = np.cumsum(nr)
    it, rk, ws = int(args.get("iteration", 0)), str(args.get("global_rank", "0")), str(args.get("world_size", "1"))
    lines = []
    tot_r = tot_c = tot_2 = 0.0
    pixels = local = 0
    for t in range(gx * gy):
        if nr[t] <= 0:
            continue
        tx, ty = t % gx, t // gx
        num_pix = (min(ty * BLOCK_Y + BLOCK_Y, H) - ty * BLOCK_Y) * (min(tx * BLOCK_X + BLOCK_X, W) - tx * BLOCK_X)
        ave_c = np.float32(nc[t]) / np.float32(num_pix)
        ave_2 = np.float32(n2[t]) / np.float32(num_pix)
        ratio = ave_2 / np.float32(nr[t]) if num_pix > 0 else np.float32(0)
        lines.append("iteration: %d, tile: (%d, %d), range: (%d, %d), num_rendered_this_tile: %d, "
                     "n_considered_per_pixel: %f, n_contrib2loss_per_pixel: %f, contrib2loss_ratio: %f"
                     % (it, ty, tx, ends[t], ends[t] - nr[t], nr[t], ave_c, ave_2, ratio))
        tot_r += float(nr[t]); tot_c += float(nc[t]); tot_2 += float(n2[t])
        pixels += num_pix
        local += 1
    lines.append("iteration: %d, global_rank: %d, world_size: %d, num_tiles: %d, num_pixels: %d, num_rendered: %d, "
                 "global_ave_n_rendered_per_pix: %f, global_ave_n_considered_per_pix: %f, "
                 "global_ave_n_contrib2loss_per_pix: %f"
                 % (it, int(rk), int(ws), local, pixels, int(tot_r), tot_r / max(local, 1), tot_c / max(pixels, 1),
                    tot_2 / max(pixels, 1)))
    path = os.path.join(str(args.get("log_folder", ".")), "n_contrib_ws=%s_rk=%s.log" % (ws, rk))
    with open(path, "a") as f:
        f.write("\n".join(lines) + "\n")


def render_gaussians_ex(background, image_height, image_width, means2D, depths, radii, conic_opacity, rgb,
                        compute_locally, viewmatrix, campos, tan_fovx, tan_fovy, all_map, render_geo, debug, args,
                        expected_instances=0, expected_longest_list=0, blend_records=None):
    """render_gaussians plus what the reference's tuple has no slot for: returns (tuple, info) with info =
    {"longest_list", "binning_capacity", "launched_ahead"}.  With expected_instances > 0 the list kernels and the
    blend are launched without waiting for the instance count, on a binning buffer laid out for
    expected_instances; info["binning_capacity"] then has to be handed to render_gaussians_backward (and to
    gs_binning_state_layout) in place of the instance count.  Results do not depend on the expectation.
    blend_records: the (P,16) operand records that preprocess_gaussians_ex wrote for exactly these inputs, all_map
    being build_all_map of the same Gaussians and camera (the blend kernels then read them and nothing is
    packed); the same tensor goes to render_gaussians_backward."""
    means2D = _f32c(means2D, "means2D")
    dev = means2D.device
    P = means2D.shape[0]
    H, W = int(image_height), int(image_width)
    f32 = dict(dtype=torch.float32, device=dev)
    i32 = dict(dtype=torch.int32, device=dev)
    tiles = ((H + BLOCK_Y - 1) // BLOCK_Y) * ((W + BLOCK_X - 1) // BLOCK_X)
    geo = bool(render_geo)
    if P == 0:
        empty = torch.empty(0, dtype=torch.uint8, device=dev)
        return ((0, torch.zeros(NUM_CHANNELS, H, W, **f32), torch.zeros(tiles, **i32), torch.zeros(tiles, **i32),
                 torch.zeros(tiles, **i32), torch.zeros(0, **i32), torch.zeros(NUM_ALL_MAP, H, W, **f32),
                 torch.zeros(1, H, W, **f32), empty, empty.clone(), empty.clone()),
                {"longest_list": 0, "binning_capacity": 0, "launched_ahead": False})
    out_color = torch.empty(NUM_CHANNELS, H, W, **f32)
    out_observe = torch.empty(P, **i32)  # cleared by the call itself
    out_all_map = torch.empty(NUM_ALL_MAP, H, W, **f32) if geo else torch.zeros(NUM_ALL_MAP, H, W, **f32)
    out_plane_depth = torch.empty(1, H, W, **f32) if geo else torch.zeros(1, H, W, **f32)
    n_render = torch.empty(tiles, **i32)
    n_consider = torch.empty(tiles, **i32)
    n_contrib = torch.empty(tiles, **i32)
    geom, binning, img = _GrowBuffer(dev), _GrowBuffer(dev), _GrowBuffer(dev)
    bg = _f32c(background, "background")
    depths, conic_opacity, rgb = _f32c(depths, "depths"), _f32c(conic_opacity, "conic_opacity"), _f32c(rgb, "rgb")
    radii = radii.contiguous()
    if radii.dtype != torch.int32:
        raise TypeError("radii must be int32")
    cl = compute_locally.contiguous()
    if cl.dtype != torch.bool or cl.numel() != tiles:
        raise RuntimeError(f"compute_locally must be a bool tensor with {tiles} elements")
    am = _f32c(all_map, "all_map") if geo else None
    want_mwd = isinstance(args, dict) and bool(args.get("max_weight_depth"))
    # (small_limit, block_records) for this call only: how the per-tile lists are built (a test hook)
    limits = args.get("tile_sort_limits") if isinstance(args, dict) else None
    options = None
    if blend_records is not None and (blend_records.shape != (P, 16) or blend_records.dtype != torch.float32
                                      or not blend_records.is_contiguous() or blend_records.device != dev):
        raise RuntimeError("blend_records must be a contiguous (P, 16) float32 tensor on the same device")
    if limits is not None or expected_instances > 0 or blend_records is not None:
        options = _n.RenderOptions(*(limits if limits is not None else (-1, -1)),
                                   expected_instances=expected_instances,
                                   expected_longest_list=expected_longest_list,
                                   blend_records=blend_records.data_ptr() if blend_records is not None else None)
    result = _n.RenderResult()
    mwd = torch.empty(1, H, W, **f32) if want_mwd else None
    # fp32 arithmetic, as `H / (2.0f * tan_fovy)` at rasterize_points.cu:328-329
    focal_y = np.float32(H) / (np.float32(2.0) * np.float32(tan_fovy))
    focal_x = np.float32(W) / (np.float32(2.0) * np.float32(tan_fovx))
    num_rendered = C.c_int(0)
    elapsed = C.c_float(0.0)
    timing = _want_timing(args)
    with torch.cuda.device(dev):
        _n.check(_lib.gs_render_forward(
            geom.callback, None, binning.callback, None, img.callback, None, P, _ptr(bg), W, H, float(focal_x),
            float(focal_y), float(W * 0.5), float(H * 0.5), _ptr(viewmatrix), _ptr(campos), _ptr(am), _ptr(means2D),
            _ptr(depths), _ptr(radii), _ptr(conic_opacity), _ptr(rgb), _ptr(cl), _ptr(out_color), _ptr(n_render),
            _ptr(n_consider), _ptr(n_contrib), _ptr(out_observe), _ptr(out_all_map), _ptr(out_plane_depth), _ptr(mwd),
            int(geo),
            int(bool(debug)), C.byref(num_rendered), C.byref(elapsed) if timing else None,
            C.byref(options) if options is not None else None, C.byref(result), _stream(dev)),
            "render_gaussians")
    _record_time(args, "forward_render_time", elapsed.value)
    if want_mwd:
        args.setdefault("stats_collector", {})["max_weight_depth"] = mwd
    if _want_tile_log(args):
        _write_tile_log(args, H, W, n_render, n_consider, n_contrib)
    info = {"longest_list": int(result.longest_list), "binning_capacity": int(result.binning_capacity),
            "launched_ahead": bool(result.launched_ahead)}
    return ((num_rendered.value, out_color, n_render, n_consider, n_contrib, out_observe, out_all_map,
             out_plane_depth, geom.release(), binning.release(), img.release()), info)


def render_gaussians_backward(background, tan_fovx, tan_fovy, all_map_pixels, all_maps, R, geomBuffer, binningBuffer,
                              imageBuffer, compute_locally, dL_dout_color, dL_dout_all_map, dL_dout_plane_depth,
                              means2D, conic_opacity, rgb, render_geo, debug, args, binning_capacity=0,
                              blend_records=None):
    """rasterize_points.cu:366-441.  Returns dL_dmeans2D as (P,2); the reference
    returns (P,3) and its Python wrapper slices [:, :2].  binning_capacity: info["binning_capacity"] of
    render_gaussians_ex when that call was given an expectation (0 otherwise); blend_records: the tensor that call
    was given, if any."""
    means2D = _f32c(means2D, "means2D")
    dev = means2D.device
    P = means2D.shape[0]
    H, W = dL_dout_color.shape[1], dL_dout_color.shape[2]
    f32 = dict(dtype=torch.float32, device=dev)
    geo = bool(render_geo)
    # every element is written by the native reduction, so no zero fill is needed
    dL_dmeans2D = torch.empty(P, 2, **f32)
    dL_dmeans2D_abs = torch.empty(P, 3, **f32)
    dL_dconic_opacity = torch.empty(P, 4, **f32)
    dL_dcolors = torch.empty(P, NUM_CHANNELS, **f32)
    dL_dall_map = torch.empty(P, NUM_ALL_MAP, **f32)
    if P != 0:
        ws_bytes = _lib.gs_render_backward_workspace_bytes(int(R))
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        bg = _f32c(background, "background")
        gpix = _f32c(dL_dout_color, "dL_dout_color")
        gmap = _f32c(dL_dout_all_map, "dL_dout_all_map") if geo else None
        gdep = _f32c(dL_dout_plane_depth, "dL_dout_plane_depth") if geo else None
        amp = _f32c(all_map_pixels, "all_map_pixels") if geo else None
        am = _f32c(all_maps, "all_maps") if geo else None
        co, col = _f32c(conic_opacity, "conic_opacity"), _f32c(rgb, "rgb")
        elapsed = C.c_float(0.0)
        timing = _want_timing(args)
        with torch.cuda.device(dev):
            _n.check(_lib.gs_render_backward(
                P, int(R), _ptr(bg), W, H, float(tan_fovx), float(tan_fovy), _ptr(geomBuffer), _ptr(binningBuffer),
                _ptr(imageBuffer), _ptr(compute_locally.contiguous()), _ptr(gpix), _ptr(gmap), _ptr(gdep),
                _ptr(dL_dmeans2D), _ptr(dL_dmeans2D_abs), _ptr(dL_dconic_opacity), _ptr(dL_dcolors), _ptr(dL_dall_map),
                _ptr(means2D), _ptr(co), _ptr(col), _ptr(am), _ptr(amp), int(geo), int(bool(debug)), _ptr(workspace),
                ws_bytes, C.byref(elapsed) if timing else None, int(binning_capacity), _ptr(blend_records),
                _stream(dev)),
                "render_gaussians_backward")
        _record_time(args, "backward_render_time", elapsed.value)
    else:
        _record_time(args, "backward_render_time", 0.0)
    return dL_dmeans2D, dL_dmeans2D_abs, dL_dconic_opacity, dL_dcolors, dL_dall_map


def rasterize_aussians_filter(means3D, scales, rotations, scale_modifier, cov3D_precomp, viewmatrix, projmatrix,
                              tan_fovx, tan_fovy, image_height, image_width, prefiltered, debug):
    """rasterize_points.cu:865-930 (the misspelt name is the reference's)."""
    if means3D.ndimension() != 2 or means3D.size(1) != 3:
        raise RuntimeError("means3D must have dimensions (num_points, 3)")
    means3D = _f32c(means3D, "means3D")
    dev = means3D.device
    P = means3D.shape[0]
    radii = torch.empty(P, dtype=torch.int32, device=dev)
    if P != 0:
        sc = _f32c(scales, "scales") if scales is not None and scales.numel() else None
        rot = _f32c(rotations, "rotations") if rotations is not None and rotations.numel() else None
        cov = _f32c(cov3D_precomp, "cov3D_precomp") if cov3D_precomp is not None and cov3D_precomp.numel() else None
        vm, pm = _f32c(viewmatrix, "viewmatrix"), _f32c(projmatrix, "projmatrix")
        with torch.cuda.device(dev):
            _n.check(_lib.gs_visible_filter(P, 0, int(image_width), int(image_height), _ptr(means3D), _ptr(sc),
                                            float(scale_modifier), _ptr(rot), _ptr(cov), _ptr(vm), _ptr(pm),
                                            float(tan_fovx), float(tan_fovy), int(bool(prefiltered)), _ptr(radii),
                                            int(bool(debug)), _stream(dev)), "rasterize_aussians_filter")
    return radii


def build_all_map(means3D, scales, rotations, viewmatrix, campos):
    """The per-Gaussian geometry channels [normal_cam(3), 1, |normal . p_cam|] that the caller of the
    reference assembles in torch between the two rasterizer ops
    (gaussian_renderer/__init__.py:1501-1518), as one kernel.  No counterpart in the reference's
    extension module."""
    means3D = _f32c(means3D, "means3D")
    dev = means3D.device
    P = means3D.shape[0]
    all_map = torch.empty(P, 5, dtype=torch.float32, device=dev)
    if P == 0:
        return all_map
    sc, rot = _f32c(scales, "scales"), _f32c(rotations, "rotations")
    vm, cp = _f32c(viewmatrix, "viewmatrix"), _f32c(campos, "campos")
    _n.check(_n.lib.gs_all_map_forward(P, _ptr(means3D), _ptr(sc), _ptr(rot), _ptr(vm), _ptr(cp), _ptr(all_map),
                                       _stream(dev)), "build_all_map")
    return all_map


def build_all_map_backward(means3D, scales, rotations, viewmatrix, campos, dL_dall_map):
    """Gradient of build_all_map with respect to means3D and (unnormalised) rotations."""
    means3D = _f32c(means3D, "means3D")
    dev = means3D.device
    P = means3D.shape[0]
    dL_dmeans3D = torch.empty(P, 3, dtype=torch.float32, device=dev)
    dL_drotations = torch.empty(P, 4, dtype=torch.float32, device=dev)
    if P == 0:
        return dL_dmeans3D, dL_drotations
    sc, rot = _f32c(scales, "scales"), _f32c(rotations, "rotations")
    vm, cp = _f32c(viewmatrix, "viewmatrix"), _f32c(campos, "campos")
    g = _f32c(dL_dall_map, "dL_dall_map")
    _n.check(_n.lib.gs_all_map_backward(P, _ptr(means3D), _ptr(sc), _ptr(rot), _ptr(vm), _ptr(cp), _ptr(g),
                                        _ptr(dL_dmeans3D), _ptr(dL_drotations), _stream(dev)),
             "build_all_map_backward")
    return dL_dmeans3D, dL_drotations


def get_distribution_strategy(*_args, **_kwargs):
    # Same behaviour as the reference (rasterizer_impl.cu:507-508).
    raise RuntimeError("getDistributionStrategy is deprecated.")


def _multi_gpu_only(name):
    def fn(*_args, **_kwargs):
        raise NotImplementedError(
            f"{name} belongs to the multi-GPU tile exchange of the reference, which this single-GPU library does not provide")
    fn.__name__ = name
    return fn


get_local2j_ids_bool = _multi_gpu_only("get_local2j_ids_bool")
get_local2j_ids_bool_adjust_mode6 = _multi_gpu_only("get_local2j_ids_bool_adjust_mode6")
get_touched_locally = _multi_gpu_only("get_touched_locally")
load_image_tiles_by_pos = _multi_gpu_only("load_image_tiles_by_pos")
set_image_tiles_by_pos = _multi_gpu_only("set_image_tiles_by_pos")
get_pixels_compute_locally_and_in_rect = _multi_gpu_only("get_pixels_compute_locally_and_in_rect")
