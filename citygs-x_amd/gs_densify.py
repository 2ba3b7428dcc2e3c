"""Densification statistics of the reference model as one call into libgsrast.so
(GaussianModel.training_statis, scene/gaussian_model.py:1181-1205)."""
import ctypes as C

import torch

import gsrast_native as _n


def _u8(mask, name):
    if mask.dtype not in (torch.bool, torch.uint8):
        raise TypeError(f"{name} must be a bool or uint8 mask, got {mask.dtype}")
    if not mask.is_cuda:
        raise RuntimeError(f"{name} must be a GPU tensor: there is no CPU path")
    return mask.contiguous().view(torch.uint8).view(-1)


def _f32(t, name):
    if t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous():
        raise RuntimeError(f"{name} must be a contiguous float32 GPU tensor")
    return t


@torch.no_grad()
def training_statis(opacity_accum, anchor_demon, offset_gradient_accum, offset_denom, n_offsets,
                    viewspace_point_grad, opacity, update_filter, offset_selection_mask, anchor_visible_mask):
    """In-place update of the four accumulators, with the arguments of GaussianModel.training_statis
    (pass `viewspace_point_tensor.grad` for `viewspace_point_grad`):

        def training_statis(self, viewspace_point_tensor, opacity, update_filter, offset_selection_mask,
                            anchor_visible_mask):
            gs_densify.training_statis(self.opacity_accum, self.anchor_demon, self.offset_gradient_accum,
                                       self.offset_denom, self.n_offsets, viewspace_point_tensor.grad, opacity,
                                       update_filter, offset_selection_mask, anchor_visible_mask)
    """
    A = opacity_accum.shape[0]
    k = int(n_offsets)
    for t, nm, n in ((opacity_accum, "opacity_accum", A), (anchor_demon, "anchor_demon", A),
                     (offset_gradient_accum, "offset_gradient_accum", A * k), (offset_denom, "offset_denom", A * k)):
        _f32(t, nm)
        if t.numel() != n:
            raise RuntimeError(f"{nm} has {t.numel()} elements, expected {n}")
    vis = _u8(anchor_visible_mask, "anchor_visible_mask")
    sel = _u8(offset_selection_mask, "offset_selection_mask")
    flt = _u8(update_filter, "update_filter")
    if vis.numel() != A:
        raise RuntimeError("anchor_visible_mask must have one entry per anchor")
    op = opacity.detach()
    op = _f32(op.contiguous(), "opacity").view(-1)
    Vk, M = sel.numel(), flt.numel()
    if op.numel() != Vk or Vk % k != 0:
        raise RuntimeError("opacity and offset_selection_mask must cover visible anchors x n_offsets candidates")
    g = viewspace_point_grad
    if g.dim() != 2 or g.shape[0] != M or g.shape[1] < 2:
        raise RuntimeError("viewspace_point_grad must be (num_selected, >=2)")
    g = _f32(g.contiguous(), "viewspace_point_grad")
    dev = opacity_accum.device
    nb = _n.lib.gs_training_stats_workspace_bytes(A, Vk)
    ws = torch.empty(nb, dtype=torch.uint8, device=dev)
    p = lambda t: C.c_void_p(t.data_ptr()) if t.numel() else None
    _n.check(_n.lib.gs_training_stats(A, k, Vk, M, p(vis), p(sel), p(flt), p(g), int(g.shape[1]), p(op),
                                      p(opacity_accum), p(anchor_demon), p(offset_gradient_accum), p(offset_denom),
                                      C.c_void_p(ws.data_ptr()), nb,
                                      C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)), "training_statis")


@torch.no_grad()
def update_max_radii(max_radii2D, radii, visibility_filter):
    """max_radii2D[visibility_filter] = max(max_radii2D[visibility_filter], radii[visibility_filter]) in place
    (densification.py:71-73), one launch."""
    _f32(max_radii2D, "max_radii2D")
    n = max_radii2D.numel()
    if radii.dtype != torch.int32 or not radii.is_cuda or radii.numel() != n:
        raise RuntimeError("radii must be an int32 GPU tensor with one entry per Gaussian")
    vis = _u8(visibility_filter, "visibility_filter")
    if vis.numel() != n:
        raise RuntimeError("visibility_filter must have one entry per Gaussian")
    dev = max_radii2D.device
    _n.check(_n.lib.gs_max_radii_update(n, C.c_void_p(radii.contiguous().data_ptr()), C.c_void_p(vis.data_ptr()),
                                        C.c_void_p(max_radii2D.data_ptr()),
                                        C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)), "update_max_radii")
    return max_radii2D
