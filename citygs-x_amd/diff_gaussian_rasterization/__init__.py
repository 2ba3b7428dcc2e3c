"""Operator API of CityGS-X's differentiable Gaussian rasterizer on MI355X.

Same names, argument order, shapes, dtypes and gradient contracts as
submodule_cityx/diff-gaussian-rasterization/diff_gaussian_rasterization/__init__.py
(GaussianRasterizationSettings :314-327, GaussianRasterizer :329-405,
preprocess op :46-146, render op :182-303), so gaussian_renderer/__init__.py
and train.py can call it unchanged.  The native side is libgsrast.so
(hand-written gfx950 kernels) reached through `_C`.

One addition: passing SH coefficients shaped (P, M, 3) as `shs` makes
preprocess evaluate colour from spherical harmonics at `sh_degree` and return
the matching dL/dshs; any other `shs` shape keeps the reference behaviour
(colour output zero, zero gradient of the same shape as `shs`).
"""
import weakref
from typing import NamedTuple

import torch
import torch.nn as nn

from . import _C

__all__ = ["GaussianRasterizationSettings", "GaussianRasterizer", "preprocess_gaussians", "render_gaussians",
           "build_all_map"]


class GaussianRasterizationSettings(NamedTuple):
    image_height: int
    image_width: int
    tanfovx: float
    tanfovy: float
    bg: torch.Tensor
    scale_modifier: float
    viewmatrix: torch.Tensor
    projmatrix: torch.Tensor
    sh_degree: int
    campos: torch.Tensor
    prefiltered: bool
    render_geo: bool
    debug: bool


# ------------------------------------------------------------ blend records --

# The blend kernels read a Gaussian's operands (centre, conic, opacity, colour, geometry channels, depth) as one
# 64-byte record.  The library packs those records itself from the separate tensors, one more pass per view, unless
# preprocess_gaussians has written them on the way: it has every value but the geometry channels at hand, and
# those it forms as build_all_map does, from the same parameters and camera.  The records travel as an attribute
# of the means2D tensor.  render_gaussians uses them only if every tensor it is given is the very tensor the
# records were written from, unmodified since (tensor identity and version counters), and, with geometry channels
# to render, if all_map is what build_all_map(..., blend_records_of=means2D) returned for the very parameter
# tensors and camera preprocess_gaussians had; otherwise the library packs.  Nothing a caller sees changes: same
# tensors, same values.

class _BlendRecords:
    __slots__ = ("records", "refs", "versions", "sources", "source_versions", "all_map_ref", "all_map_version")

    def __init__(self, records, parts, sources):
        self.records = records
        self.refs = [weakref.ref(t) for t in parts]
        self.versions = [t._version for t in parts]
        # means3D, scales, rotations, viewmatrix, campos as preprocess_gaussians had them
        self.sources = [weakref.ref(t) for t in sources]
        self.source_versions = [t._version for t in sources]
        self.all_map_ref = None
        self.all_map_version = -1

    def same_sources(self, sources):
        return all(ref() is t and t._version == v for ref, v, t in zip(self.sources, self.source_versions, sources))

    def usable(self, parts, all_maps, render_geo):
        for ref, version, t in zip(self.refs, self.versions, parts):
            if ref() is not t or t._version != version:
                return False
        if render_geo and (self.all_map_ref is None or self.all_map_ref() is not all_maps
                           or all_maps._version != self.all_map_version):
            return False
        return True


_linked_all_map_seen = [False]  # the caller builds all_map with blend_records_of=...: records are worth starting
_pending_blend = [None]         # from _PreprocessGaussians.forward to the wrapper that tags its outputs


def _records_wanted(rs, P, device):
    """Whether preprocess should write the records: the last view of this image size had enough instances per
    Gaussian for records to pay (written on the way they cost about a third of the library's packing pass, which
    pays from 0.8 instances per Gaussian), and render_gaussians will be able to use them (no geometry channels to
    render, or the caller builds them through build_all_map(..., blend_records_of=means2D))."""
    seen = _expectations.get((rs.image_height, rs.image_width, device))
    if seen is None or seen[0] * 10 <= P * 3:
        return False
    return (not rs.render_geo) or _linked_all_map_seen[0]


# --------------------------------------------------------------- preprocess --

class _PreprocessGaussians(torch.autograd.Function):
    @staticmethod
    def forward(ctx, means3D, scales, rotations, sh, opacities, raster_settings, cuda_args):
        rs = raster_settings
        # (when a backward pass can follow, the forward kernel also leaves the colours' derivative with respect to
        # the view direction, nine numbers per Gaussian, which is all the backward kernel needs the coefficients for)
        P = means3D.shape[0]
        records = (torch.empty(P, 16, dtype=torch.float32, device=means3D.device)
                   if P > 0 and _records_wanted(rs, P, means3D.device) else None)
        (num_rendered, means2D, depths, radii, cov3D, conic_opacity, rgb, clamped), ddir = _C.preprocess_gaussians_ex(
            means3D, scales, rotations, sh, opacities, rs.scale_modifier, rs.viewmatrix, rs.projmatrix, rs.tanfovx,
            rs.tanfovy, rs.image_height, rs.image_width, rs.sh_degree, rs.campos, rs.prefiltered, rs.debug, cuda_args,
            want_direction_derivative=any(ctx.needs_input_grad[:5]), want_cov3D=False, blend_records=records)
        _pending_blend[0] = ((records, (means3D, scales, rotations, rs.viewmatrix, rs.campos))
                             if records is not None else None)
        # (cov3D is None: the backward kernel forms the covariances again from scales and rotations, which it reads
        # anyway, instead of both passes moving 24 bytes per Gaussian)
        ctx.raster_settings = rs
        ctx.cuda_args = cuda_args
        ctx.num_rendered = num_rendered
        ctx.has_ddir = ddir is not None
        ctx.save_for_backward(means3D, scales, rotations, sh, radii, cov3D, clamped,
                              *([ddir] if ddir is not None else []))
        ctx.mark_non_differentiable(radii, depths)
        # no zero tensors for the outputs nobody differentiates (radii, depths): backward fills in what it needs
        ctx.set_materialize_grads(False)
        return means2D, rgb, conic_opacity, radii, depths

    @staticmethod
    def backward(ctx, grad_means2D, grad_rgb, grad_conic_opacity, grad_radii, grad_depths):
        rs = ctx.raster_settings
        means3D, scales, rotations, sh, radii, cov3D, clamped = ctx.saved_tensors[:7]
        ddir = ctx.saved_tensors[7] if ctx.has_ddir else None
        P = means3D.shape[0]
        if grad_means2D is None:
            grad_means2D = means3D.new_zeros(P, 2)
        if grad_rgb is None:
            grad_rgb = means3D.new_zeros(P, 3)
        if grad_conic_opacity is None:
            grad_conic_opacity = means3D.new_zeros(P, 4)
        dL_dmeans3D, dL_dscales, dL_drotations, dL_dsh, dL_dopacity = _C.preprocess_gaussians_backward(
            radii, cov3D, clamped, means3D, scales, rotations, sh, rs.scale_modifier, rs.viewmatrix, rs.projmatrix,
            rs.tanfovx, rs.tanfovy, rs.image_height, rs.image_width, rs.sh_degree, rs.campos, grad_means2D,
            grad_conic_opacity, grad_rgb, ctx.num_rendered, rs.debug, ctx.cuda_args, dcolor_ddir=ddir)
        if dL_dsh.shape != sh.shape:
            dL_dsh = torch.zeros_like(sh)
        return dL_dmeans3D, dL_dscales, dL_drotations, dL_dsh, dL_dopacity, None, None


def preprocess_gaussians(means3D, scales, rotations, sh, opacities, raster_settings, cuda_args):
    _pending_blend[0] = None
    means2D, rgb, conic_opacity, radii, depths = _PreprocessGaussians.apply(means3D, scales, rotations, sh, opacities,
                                                                            raster_settings, cuda_args)
    pending, _pending_blend[0] = _pending_blend[0], None
    if pending is not None:
        means2D._gs_blend = _BlendRecords(pending[0], (means2D, conic_opacity, rgb, depths), pending[1])
    return means2D, rgb, conic_opacity, radii, depths


# ------------------------------------------------------------------- render --

# What the last view of a given image size needed, (instances, longest list) keyed by (height, width, device): the
# next view of that size is launched without waiting for its instance count, on buffers sized for these figures plus
# a margin (a training loop renders thousands of similar views; the number of Gaussians changes at every
# densification, so it is not part of the key).  Only the time depends on it, never a result; a stale or missing
# entry costs one ordinary call.  A handful of image sizes at most are alive in a run: the oldest entry goes
# when there are more than _MAX_EXPECTATIONS.
_expectations = {}
_MARGIN = 1.25
_MAX_EXPECTATIONS = 16


def _expectation(key):
    seen = _expectations.get(key)
    if seen is None:
        return 0, 0
    instances, longest = seen
    if longest <= 0:
        return 0, 0  # a view without per-tile lists (a tile grid too large for them): nothing to gain
    # whole variants of the register sort (256 ... 2048 records per list), so that a slightly longer list still
    # fits; beyond them any length (0): the radix sort's kernels are launched as well
    cap = 256
    while cap < longest * _MARGIN:
        cap *= 2
    return int(instances * _MARGIN) + 65536, (cap if cap <= 2048 else 0)


def _remember(key, instances, longest):
    _expectations.pop(key, None)  # (re-inserted at the end: the dict keeps insertion order)
    _expectations[key] = (instances, longest)
    while len(_expectations) > _MAX_EXPECTATIONS:
        _expectations.pop(next(iter(_expectations)))


class _RenderGaussians(torch.autograd.Function):
    @staticmethod
    def forward(ctx, means2D, means2D_abs, conic_opacity, rgb, all_maps, depths, radii, compute_locally,
                extended_compute_locally, raster_settings, cuda_args):
        rs = raster_settings
        avoid = bool(cuda_args.get("avoid_pixel_all2all", False)) if cuda_args is not None else False
        mask = extended_compute_locally if avoid else compute_locally
        key = (rs.image_height, rs.image_width, means2D.device)
        expected_instances, expected_longest = _expectation(key)
        blend = getattr(means2D, "_gs_blend", None)
        records = (blend.records if blend is not None and blend.usable((means2D, conic_opacity, rgb, depths), all_maps,
                                                                       rs.render_geo) else None)
        if blend is not None and records is None and rs.render_geo:
            # records were written and cannot be used: the caller does not (or no longer) build all_map through
            # build_all_map(..., blend_records_of=means2D); stop writing them until it does
            _linked_all_map_seen[0] = False
        ((num_rendered, color, n_render, n_consider, n_contrib, out_observe, out_all_map, out_plane_depth, geomBuffer,
          binningBuffer, imgBuffer), info) = _C.render_gaussians_ex(
            rs.bg, rs.image_height, rs.image_width, means2D, depths, radii, conic_opacity, rgb, mask, rs.viewmatrix,
            rs.campos, rs.tanfovx, rs.tanfovy, all_maps, rs.render_geo, rs.debug, cuda_args,
            expected_instances=expected_instances, expected_longest_list=expected_longest, blend_records=records)
        ctx.blend_records = records
        if means2D.shape[0] > 0:
            _remember(key, num_rendered, info["longest_list"])
        if isinstance(cuda_args, dict) and isinstance(cuda_args.get("stats_collector"), dict):
            # (beside the reference's timing keys: whether this view's list kernels ran ahead of its instance count)
            cuda_args["stats_collector"]["launched_ahead"] = info["launched_ahead"]
            cuda_args["stats_collector"]["num_rendered"] = num_rendered
        ctx.binning_capacity = info["binning_capacity"]
        ctx.raster_settings = rs
        ctx.cuda_args = cuda_args
        ctx.num_rendered = num_rendered
        ctx.save_for_backward(means2D, conic_opacity, rgb, all_maps, out_all_map, geomBuffer, binningBuffer, imgBuffer,
                              compute_locally)
        ctx.mark_non_differentiable(n_render, n_consider, n_contrib, out_observe)
        ctx.set_materialize_grads(False)  # the four integer outputs never get a zero "gradient" allocated
        return color, n_render, n_consider, n_contrib, out_observe, out_all_map, out_plane_depth

    @staticmethod
    def backward(ctx, grad_color, grad_n_render, grad_n_consider, grad_n_contrib, grad_out_observe, grad_out_all_map,
                 grad_out_plane_depth):
        rs = ctx.raster_settings
        (means2D, conic_opacity, rgb, all_maps, all_map_pixels, geomBuffer, binningBuffer, imgBuffer,
         compute_locally) = ctx.saved_tensors
        if grad_color is None:
            grad_color = torch.zeros_like(all_map_pixels[:3])
        if rs.render_geo:
            if grad_out_all_map is None:
                grad_out_all_map = torch.zeros_like(all_map_pixels)
            if grad_out_plane_depth is None:
                grad_out_plane_depth = torch.zeros_like(all_map_pixels[:1])
        dL_dmeans2D, dL_dmeans2D_abs, dL_dconic_opacity, dL_dcolors, dL_dall_map = _C.render_gaussians_backward(
            rs.bg, rs.tanfovx, rs.tanfovy, all_map_pixels, all_maps, ctx.num_rendered, geomBuffer, binningBuffer,
            imgBuffer, compute_locally, grad_color, grad_out_all_map, grad_out_plane_depth, means2D, conic_opacity,
            rgb, rs.render_geo, rs.debug, ctx.cuda_args, binning_capacity=ctx.binning_capacity,
            blend_records=ctx.blend_records)
        return (dL_dmeans2D, dL_dmeans2D_abs, dL_dconic_opacity, dL_dcolors, dL_dall_map, None, None, None, None, None,
                None)


def render_gaussians(means2D, means2D_abs, conic_opacity, rgb, all_map, depths, radii, compute_locally,
                     extended_compute_locally, raster_settings, cuda_args):
    return _RenderGaussians.apply(means2D, means2D_abs, conic_opacity, rgb, all_map, depths, radii, compute_locally,
                                  extended_compute_locally, raster_settings, cuda_args)


# ------------------------------------------------------------------ all_map --

class _BuildAllMap(torch.autograd.Function):
    @staticmethod
    def forward(ctx, means3D, scales, rotations, viewmatrix, campos):
        ctx.save_for_backward(means3D, scales, rotations, viewmatrix, campos)
        return _C.build_all_map(means3D, scales, rotations, viewmatrix, campos)

    @staticmethod
    def backward(ctx, grad_all_map):
        means3D, scales, rotations, viewmatrix, campos = ctx.saved_tensors
        dL_dmeans3D, dL_drotations = _C.build_all_map_backward(means3D, scales, rotations, viewmatrix, campos,
                                                               grad_all_map)
        return dL_dmeans3D, None, dL_drotations, None, None


def build_all_map(means3D, scales, rotations, viewmatrix, campos, blend_records_of=None):
    """[normal in the camera frame, 1, |normal . p_cam|] per Gaussian: a drop-in for the torch lines
    gaussian_renderer/__init__.py:1501-1518 (pass the camera's world_view_transform and camera_center).
    Differentiable in means3D and rotations, like those lines; `scales` only picks the axis.
    blend_records_of (optional): the means2D tensor preprocess_gaussians returned for the same parameter tensors
    and camera (the settings' viewmatrix and campos tensors).  preprocess_gaussians then writes the blend kernels'
    operand records with these very channels in them (from the next view on), and render_gaussians, given these
    very tensors, skips the pass that packs them.  The returned tensor is the same either way."""
    all_map = _BuildAllMap.apply(means3D, scales, rotations, viewmatrix, campos)
    if blend_records_of is not None:
        _linked_all_map_seen[0] = True
        blend = getattr(blend_records_of, "_gs_blend", None)
        if blend is not None and blend.same_sources((means3D, scales, rotations, viewmatrix, campos)):
            blend.all_map_ref = weakref.ref(all_map)
            blend.all_map_version = all_map._version
    return all_map


# ------------------------------------------------------------------- module --

class GaussianRasterizer(nn.Module):
    def __init__(self, raster_settings):
        super().__init__()
        self.raster_settings = raster_settings

    def markVisible(self, positions):
        """Boolean mask of points in front of the camera."""
        with torch.no_grad():
            rs = self.raster_settings
            return _C.mark_visible(positions, rs.viewmatrix, rs.projmatrix)

    def preprocess_gaussians(self, means3D, scales, rotations, shs, opacities, cuda_args=None):
        return preprocess_gaussians(means3D, scales, rotations, shs, opacities, self.raster_settings, cuda_args)

    def visible_filter(self, means3D, scales=None, rotations=None, cov3D_precomp=None):
        rs = self.raster_settings
        if scales is None:
            scales = torch.Tensor([])
        if rotations is None:
            rotations = torch.Tensor([])
        if cov3D_precomp is None:
            cov3D_precomp = torch.Tensor([])
        with torch.no_grad():
            return _C.rasterize_aussians_filter(means3D, scales, rotations, rs.scale_modifier, cov3D_precomp,
                                                rs.viewmatrix, rs.projmatrix, rs.tanfovx, rs.tanfovy, rs.image_height,
                                                rs.image_width, rs.prefiltered, rs.debug)

    def render_gaussians(self, means2D, means2D_abs, conic_opacity, rgb, all_map, depths, radii, compute_locally,
                         extended_compute_locally, cuda_args=None):
        return render_gaussians(means2D, means2D_abs, conic_opacity, rgb, all_map, depths, radii, compute_locally,
                                extended_compute_locally, self.raster_settings, cuda_args)
