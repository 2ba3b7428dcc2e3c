"""Neural-Gaussian generation of the reference, generate_neural_gaussians (gaussian_renderer/__init__.py:789-899),
as three kernel launches forward (opacity MLP, scan, color/cov MLPs with the post-processing) and two backward,
in libgsrast.so.  The fused operator is the reference's default model configuration (arguments/__init__.py:94-124):
feat_dim 32, inputs [feature, view direction]; the operator also takes the optional distance and level inputs of the
three MLPs (add_opacity_dist, add_color_dist, add_cov_dist, add_level) and the per-anchor opacity factor of dist2level
'progressive'; the drop-in function also serves the appearance embedding and the feature bank, which reduce to it."""
import ctypes as C

import torch

import gsrast_native as _n


def _p(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _f32(t, name, shape):
    if t.dtype != torch.float32:
        raise TypeError(f"{name} must be float32, got {t.dtype}")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a GPU tensor: there is no CPU path")
    if tuple(t.shape) != tuple(shape):
        raise RuntimeError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    return t.contiguous()


def _table(tensors):
    arr = (C.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])
    return arr


def _param_shapes(k, input_flags=0):
    shapes = []
    for m, out in enumerate((k, 3 * k, 7 * k)):
        shapes += [(32, 35 + ((input_flags >> m) & 1) + ((input_flags >> 3) & 1)), (32,), (out, 32), (out,)]
    return shapes


class _NeuralGaussians(torch.autograd.Function):
    @staticmethod
    def forward(ctx, anchor, feat, offsets, scaling, campos, opacity_scale, level, input_flags, *params):
        if len(params) != 12:
            raise RuntimeError("expected W1, b1, W2, b2 of the opacity, color and cov MLPs (12 tensors)")
        N = anchor.shape[0]
        if offsets.dim() != 3:
            raise RuntimeError("offsets must be (anchors, n_offsets, 3)")
        k = offsets.shape[1]
        if not _n.lib.gs_neural_supported(k):
            raise NotImplementedError(f"n_offsets = {k} is not among the values the kernels are built for")
        anchor, feat = _f32(anchor, "anchor", (N, 3)), _f32(feat, "feat", (N, 32))
        offsets, scaling = _f32(offsets, "offsets", (N, k, 3)), _f32(scaling, "scaling", (N, 6))
        campos = _f32(campos, "camera_center", (3,))
        if opacity_scale is not None:
            opacity_scale = _f32(opacity_scale.detach(), "opacity_scale", (N,))
        if input_flags & 8:
            if level is None:
                raise RuntimeError("input_flags asks for the level input")
            level = _f32(level.detach().reshape(-1), "level", (N,))
        else:
            level = None
        params = [_f32(p, f"MLP parameter {i}", s)
                  for i, (p, s) in enumerate(zip(params, _param_shapes(k, input_flags)))]
        dev = anchor.device
        stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
        neural_opacity = torch.empty(N * k, 1, dtype=torch.float32, device=dev)
        # with a factor on the opacity the backward pass needs the MLP's own output as well
        opacity_tanh = torch.empty(N * k, dtype=torch.float32, device=dev) if opacity_scale is not None else None
        mask = torch.empty(N * k, dtype=torch.bool, device=dev)
        first = torch.empty(max(N, 1), dtype=torch.int32, device=dev)
        ws_bytes = _n.lib.gs_neural_workspace_bytes(N, k)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        table = _table(params)
        S = C.c_int64(0)
        _n.check(_n.lib.gs_neural_opacity_forward(N, k, _p(anchor), _p(feat), _p(campos), table,
                                                  _p(opacity_scale), _p(level), input_flags,
                                                  _p(neural_opacity), _p(opacity_tanh), _p(mask), _p(first), _p(ws), ws_bytes,
                                                  C.byref(S), stream),
                 "generate_neural_gaussians")
        S = S.value
        xyz, color = torch.empty(S, 3, device=dev), torch.empty(S, 3, device=dev)
        opacity, scal = torch.empty(S, 1, device=dev), torch.empty(S, 3, device=dev)
        rot, aux = torch.empty(S, 4, device=dev), torch.empty(S, 4, device=dev)
        _n.check(_n.lib.gs_neural_gaussians_forward(N, k, S, _p(anchor), _p(feat), _p(offsets), _p(scaling),
                                                    _p(campos), _p(level), _p(neural_opacity), _p(first), _p(ws),
                                                    ws_bytes,
                                                    _p(xyz), _p(color), _p(opacity), _p(scal), _p(rot), _p(aux),
                                                    stream), "generate_neural_gaussians")
        ctx.save_for_backward(anchor, feat, offsets, scaling, campos, neural_opacity, first, color, rot, aux, *params)
        ctx.sizes = (N, k, S)
        ctx.opacity_scale = opacity_scale  # carries no gradient (a buffer of the model)
        ctx.level, ctx.input_flags, ctx.opacity_tanh = level, input_flags, opacity_tanh
        ctx.mark_non_differentiable(neural_opacity, mask)
        ctx.set_materialize_grads(False)
        return xyz, color, opacity, scal, rot, neural_opacity, mask

    @staticmethod
    def backward(ctx, g_xyz, g_color, g_opacity, g_scal, g_rot, _g_nop, _g_mask):
        anchor, feat, offsets, scaling, campos, neural_opacity, first, color, rot, aux, *params = ctx.saved_tensors
        N, k, S = ctx.sizes
        dev = anchor.device
        ups = []
        for g, c in ((g_xyz, 3), (g_color, 3), (g_opacity, 1), (g_scal, 3), (g_rot, 4)):
            ups.append(torch.zeros(S, c, device=dev) if g is None else _f32(g, "upstream gradient", (S, c)))
        d_anchor, d_feat = torch.empty_like(anchor), torch.empty_like(feat)
        d_offsets, d_scaling = torch.empty_like(offsets), torch.empty_like(scaling)
        d_params = [torch.empty_like(p) for p in params]
        ws_bytes = _n.lib.gs_neural_backward_workspace_bytes(N, k)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
        _n.check(_n.lib.gs_neural_backward(N, k, S, _p(anchor), _p(feat), _p(offsets), _p(scaling), _p(campos),
                                           _table(params),
                                           _p(ctx.opacity_scale), _p(ctx.level), ctx.input_flags,
                                           _p(neural_opacity), _p(ctx.opacity_tanh), _p(first), _p(color), _p(rot),
                                           _p(aux),
                                           *[_p(u) for u in ups], _p(d_anchor), _p(d_feat), _p(d_offsets),
                                           _p(d_scaling), _table(d_params), _p(ws), ws_bytes, stream),
                 "generate_neural_gaussians backward")
        return (d_anchor, d_feat, d_offsets, d_scaling, None, None, None, None, *d_params)


def neural_gaussians(anchor, feat, offsets, scaling, camera_center, mlp_opacity, mlp_color, mlp_cov,
                     opacity_scale=None, level=None, input_flags=0):
    """The body of generate_neural_gaussians after the visible_mask gathers (gaussian_renderer/__init__.py:800-896).
    anchor (N,3), feat (N,32), offsets (N,k,3), scaling (N,6) = get_scaling, camera_center (3); each mlp_* is
    (W1, b1, W2, b2) as nn.Linear holds them; opacity_scale (N), if given, multiplies the opacity MLP's output per
    anchor (:844-848); input_flags (add_opacity_dist = 1, add_color_dist = 2, add_cov_dist = 4: that MLP's W1 has a
    column for the distance; add_level = 8: all three have a last column for level (N), :824-877).
    Returns (xyz, color, opacity, scaling, rot, neural_opacity, mask);
    differentiable in everything but the camera centre; neural_opacity and mask carry no gradient (the reference
    uses them detached, scene/gaussian_model.py:1183)."""
    return _NeuralGaussians.apply(anchor, feat, offsets, scaling, camera_center, opacity_scale, level, input_flags,
                                  *mlp_opacity, *mlp_color, *mlp_cov)


def _linear_pair(seq):
    """(W1, b1, W2, b2) of a Sequential(Linear, ReLU, Linear[, activation]) (scene/gaussian_model.py:131-149)."""
    return seq[0].weight, seq[0].bias, seq[2].weight, seq[2].bias


def generate_neural_gaussians(viewpoint_camera, pc, visible_mask=None, is_training=False, ape_code=-1):
    """Same signature and results as gaussian_renderer/__init__.py:789-899.  Served: the default configuration,
    the appearance embedding (appearance_dim > 0: every anchor of a view gets the same embedding row, :830-836,
    :866-868, so its part of the first color layer is a per-view addition to that layer's bias) and the feature
    bank (use_feat_bank, :809-823: the view-dependent mix of the feature's resolutions is a few torch lines ahead
    of the fused operator), dist2level 'progressive' (:844-848: the opacity of an anchor in transition is scaled
    by its progress ratio) and the distance / level inputs of the MLPs (add_opacity_dist, add_color_dist,
    add_cov_dist, add_level, :824-829, :839-877)."""
    input_flags = ((1 if pc.add_opacity_dist else 0) | (2 if pc.add_color_dist else 0) | (4 if pc.add_cov_dist else 0)
                   | (8 if pc.add_level else 0))
    level = None
    progressive = pc.dist2level == "progressive"
    opacity_scale = None
    if visible_mask is None:
        anchor, feat, offsets, scaling = pc.get_anchor, pc.get_anchor_feat, pc._offset, pc.get_scaling
        if pc.add_level:
            level = pc.get_level.reshape(-1).float()
        if progressive:
            opacity_scale = torch.where(pc.transition_mask, pc._prog_ratio.reshape(-1),
                                        torch.ones_like(pc._prog_ratio.reshape(-1)))
    else:
        # one nonzero() (one host synchronisation) serves the four gathers; x[visible_mask] would run it four times
        idx = visible_mask.nonzero(as_tuple=True)[0]
        anchor, feat = pc.get_anchor.index_select(0, idx), pc.get_anchor_feat.index_select(0, idx)
        offsets, scaling = pc._offset.index_select(0, idx), pc.get_scaling.index_select(0, idx)
        if pc.add_level:
            level = pc.get_level.reshape(-1).index_select(0, idx).float()
        if progressive:
            prog = pc._prog_ratio.reshape(-1).index_select(0, idx)
            opacity_scale = torch.where(pc.transition_mask.index_select(0, idx), prog, torch.ones_like(prog))
    if pc.use_feat_bank:
        ob_view = anchor - viewpoint_camera.camera_center
        ob_view = ob_view / ob_view.norm(dim=1, keepdim=True)
        cat_view = torch.cat([ob_view, level.unsqueeze(1)], dim=1) if pc.add_level else ob_view
        bank_weight = pc.get_featurebank_mlp(cat_view).unsqueeze(dim=1)  # [n, 1, 3]
        f = feat.unsqueeze(dim=-1)
        f = f[:, ::4, :1].repeat([1, 4, 1]) * bank_weight[:, :, :1] + \
            f[:, ::2, :1].repeat([1, 2, 1]) * bank_weight[:, :, 1:2] + \
            f[:, ::1, :1] * bank_weight[:, :, 2:]
        feat = f.squeeze(dim=-1)
    color_mlp = _linear_pair(pc.get_color_mlp)
    if pc.appearance_dim > 0:
        cam_id = viewpoint_camera.uid if (is_training or ape_code < 0) else ape_code[0]
        row = pc.get_appearance(torch.tensor([cam_id], dtype=torch.long, device=anchor.device))[0]
        W1 = color_mlp[0]
        base = 35 + (1 if pc.add_color_dist else 0) + (1 if pc.add_level else 0)  # the embedding's first column
        color_mlp = (W1[:, :base].contiguous(), color_mlp[1] + W1[:, base:] @ row, color_mlp[2], color_mlp[3])
    out = neural_gaussians(anchor, feat, offsets, scaling, viewpoint_camera.camera_center,
                           _linear_pair(pc.get_opacity_mlp), color_mlp, _linear_pair(pc.get_cov_mlp), opacity_scale,
                           level, input_flags)
    return out if is_training else out[:5]
