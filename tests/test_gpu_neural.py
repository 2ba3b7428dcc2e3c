"""Neural-Gaussian generation (gaussian_renderer/__init__.py:789-899) on the GPU against the CPU oracle, and at
a training-sized anchor count against the same statements run by torch on the device."""
import numpy as np
import pytest
import torch

import gs_scenes

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _rel(a, b):
    a, b = np.asarray(a, np.float64).ravel(), np.asarray(b, np.float64).ravel()
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


def _to_dev(s, grad=False):
    leaf = lambda t: t.to(DEV).requires_grad_(grad)
    mlps = [tuple(leaf(x) for x in m) for m in s["mlps"]]
    return leaf(s["anchor"]), leaf(s["feat"]), leaf(s["offsets"]), leaf(s["scaling"]), s["campos"].to(DEV), mlps


def _np_args(s):
    n = lambda t: t.numpy()
    return (n(s["anchor"]), n(s["feat"]), n(s["offsets"]), n(s["scaling"]), n(s["campos"]),
            [tuple(n(x) for x in m) for m in s["mlps"]])


def _dense(rows, mask, width):
    """Compacted rows scattered back to their (anchor, offset) slots."""
    out = np.zeros((mask.shape[0], width), np.float64)
    out[mask] = np.asarray(rows, np.float64).reshape(-1, width)
    return out


@pytest.mark.parametrize("N,k,seed", [(1000, 10, 0), (33, 10, 1), (1, 10, 2), (300, 5, 3), (97, 4, 4), (64, 16, 5),
                                      (129, 1, 6), (70, 12, 7), (40, 3, 8), (45, 8, 9), (31, 2, 10), (200, 6, 11),
                                      (90, 7, 12), (77, 9, 13), (66, 11, 14), (130, 13, 15), (55, 14, 16),
                                      (100, 15, 17)])
def test_forward_and_backward_match_oracle(orc, N, k, seed):
    from gs_neural import neural_gaussians
    s = gs_scenes.make_anchor_scene(N, k, seed)
    anchor, feat, offsets, scaling, campos, mlps = _to_dev(s, grad=True)
    out = neural_gaussians(anchor, feat, offsets, scaling, campos, *mlps)
    want = orc.neural_gaussians_fwd(*_np_args(s))
    got = [o.detach().cpu().numpy() for o in out]
    assert got[5].shape == (N * k, 1) and got[6].shape == (N * k,) and got[6].dtype == np.bool_
    assert np.abs(got[5] - want[5]).max() <= 2e-6
    # the selection may differ only where the opacity is zero to rounding
    differ = got[6] != want[6]
    assert np.abs(want[5].ravel()[differ]).max(initial=0.0) <= 2e-6
    assert np.array_equal(got[6], got[5].ravel() > 0)
    S = int(got[6].sum())
    for g, c in zip(got[:5], (3, 3, 1, 3, 4)):
        assert g.shape == (S, c)
    both = got[6] & want[6]
    for g, w, c in zip(got[:5], want[:5], (3, 3, 1, 3, 4)):
        assert _rel(_dense(g, got[6], c)[both], _dense(w, want[6], c)[both]) <= 5e-6
    if differ.any():
        return  # (not seen with these seeds) the gradient comparison needs the same selection
    gen = torch.Generator().manual_seed(seed)
    ups = [torch.randn(S, c, generator=gen) for c in (3, 3, 1, 3, 4)]
    sum((o * u.to(DEV)).sum() for o, u in zip(out[:5], ups)).backward()
    wd = orc.neural_gaussians_bwd(*_np_args(s), *[u.numpy() for u in ups])
    for name, t, w in zip(("anchor", "feat", "offsets", "scaling"), (anchor, feat, offsets, scaling), wd[:4]):
        assert t.grad.shape == t.shape
        assert _rel(t.grad.cpu().numpy(), w) <= 1e-5, name
    flat = [x for m in mlps for x in m]
    for i, (t, w) in enumerate(zip(flat, wd[4])):
        assert _rel(t.grad.cpu().numpy(), w) <= 2e-5, i


def _prog(N, seed):
    gen = torch.Generator().manual_seed(100 + seed)
    prog = torch.rand(N, 1, generator=gen) * 0.98 + 0.01
    prog[torch.rand(N, generator=gen) < 0.4] = 1.0
    prog[torch.rand(N, generator=gen) < 0.1] = 0.0
    return prog


@pytest.mark.parametrize("N,k,seed", [(700, 10, 20), (45, 5, 21), (130, 16, 22)])
def test_progressive_opacity_factor_matches_oracle(orc, N, k, seed):
    """dist2level 'progressive' (gaussian_renderer/__init__.py:844-848): a per-anchor factor on the opacity."""
    from gs_neural import neural_gaussians
    s = gs_scenes.make_anchor_scene(N, k, seed)
    prog = _prog(N, seed)
    anchor, feat, offsets, scaling, campos, mlps = _to_dev(s, grad=True)
    out = neural_gaussians(anchor, feat, offsets, scaling, campos, *mlps, opacity_scale=prog.reshape(-1).to(DEV))
    want = orc.neural_gaussians_fwd(*_np_args(s), prog=prog.numpy())
    got = [o.detach().cpu().numpy() for o in out]
    assert np.abs(got[5] - want[5]).max() <= 2e-6
    assert np.array_equal(got[6], want[6])
    assert not got[6].reshape(N, k)[prog.numpy().ravel() == 0].any()
    for g, w in zip(got[:5], want[:5]):
        assert _rel(g, w) <= 5e-6
    S = int(got[6].sum())
    gen = torch.Generator().manual_seed(seed)
    ups = [torch.randn(S, c, generator=gen) for c in (3, 3, 1, 3, 4)]
    sum((o * u.to(DEV)).sum() for o, u in zip(out[:5], ups)).backward()
    wd = orc.neural_gaussians_bwd(*_np_args(s), *[u.numpy() for u in ups], prog=prog.numpy())
    for name, t, w in zip(("anchor", "feat", "offsets", "scaling"), (anchor, feat, offsets, scaling), wd[:4]):
        assert _rel(t.grad.cpu().numpy(), w) <= 1e-5, name
    flat = [x for m in mlps for x in m]
    for i, (t, w) in enumerate(zip(flat, wd[4])):
        assert _rel(t.grad.cpu().numpy(), w) <= 2e-5, i


@pytest.mark.parametrize("N,k,seed,flags", [(600, 10, 30, 15), (100, 5, 31, 1), (100, 4, 32, 2), (100, 3, 33, 4),
                                            (333, 10, 34, 8), (150, 16, 35, 13), (64, 1, 36, 7)])
def test_distance_and_level_inputs_match_oracle(orc, N, k, seed, flags):
    """add_opacity_dist = 1, add_color_dist = 2, add_cov_dist = 4, add_level = 8
    (gaussian_renderer/__init__.py:824-829, :839-877)."""
    from gs_neural import neural_gaussians
    s = gs_scenes.make_anchor_scene(N, k, seed, input_flags=flags)
    anchor, feat, offsets, scaling, campos, mlps = _to_dev(s, grad=True)
    out = neural_gaussians(anchor, feat, offsets, scaling, campos, *mlps, level=s["level"].to(DEV),
                           input_flags=flags)
    want = orc.neural_gaussians_fwd(*_np_args(s), level=s["level"].numpy(), input_flags=flags)
    got = [o.detach().cpu().numpy() for o in out]
    assert np.abs(got[5] - want[5]).max() <= 5e-6
    differ = got[6] != want[6]
    assert np.abs(want[5].ravel()[differ]).max(initial=0.0) <= 5e-6
    both = got[6] & want[6]
    for g, w, c in zip(got[:5], want[:5], (3, 3, 1, 3, 4)):
        assert _rel(_dense(g, got[6], c)[both], _dense(w, want[6], c)[both]) <= 1e-5
    if differ.any():
        return
    S = int(got[6].sum())
    gen = torch.Generator().manual_seed(seed)
    ups = [torch.randn(S, c, generator=gen) for c in (3, 3, 1, 3, 4)]
    sum((o * u.to(DEV)).sum() for o, u in zip(out[:5], ups)).backward()
    wd = orc.neural_gaussians_bwd(*_np_args(s), *[u.numpy() for u in ups], level=s["level"].numpy(),
                                  input_flags=flags)
    for name, t, w in zip(("anchor", "feat", "offsets", "scaling"), (anchor, feat, offsets, scaling), wd[:4]):
        assert t.grad.shape == t.shape
        assert _rel(t.grad.cpu().numpy(), w) <= 2e-5, name
    flat = [x for m in mlps for x in m]
    for i, (t, w) in enumerate(zip(flat, wd[4])):
        assert t.grad.shape == t.shape
        assert _rel(t.grad.cpu().numpy(), w) <= 3e-5, i


def test_progressive_factor_with_saturated_opacity_units(orc):
    """With the distance as an input the opacity MLP's outputs saturate (tanh within an ulp or two of 1), where
    1 - tanh^2 is a few 1e-7: the backward pass must take it from the tanh the forward pass computed, not from
    opacity / factor.  The opacity MLP's gradients are tiny here and still the oracle's."""
    from gs_neural import neural_gaussians
    N, k, flags, seed = 31, 9, 7, 695985
    s = gs_scenes.make_anchor_scene(N, k, seed, input_flags=flags)
    gen = torch.Generator().manual_seed(seed)
    prog = torch.rand(N, 1, generator=gen) * 0.98 + 0.01
    prog[torch.rand(N, generator=gen) < 0.3] = 1.0
    prog[torch.rand(N, generator=gen) < 0.1] = 0.0
    anchor, feat, offsets, scaling, campos, mlps = _to_dev(s, grad=True)
    out = neural_gaussians(anchor, feat, offsets, scaling, campos, *mlps, opacity_scale=prog.reshape(-1).to(DEV),
                           level=s["level"].to(DEV), input_flags=flags)
    kw = dict(prog=prog.numpy(), level=s["level"].numpy(), input_flags=flags)
    want = orc.neural_gaussians_fwd(*_np_args(s), **kw)
    got = [o.detach().cpu().numpy() for o in out]
    assert np.array_equal(got[6], want[6])
    th = want[5].reshape(N, k) / np.where(prog.numpy() > 0, prog.numpy(), 1.0)
    assert (np.abs(th) > 1 - 1e-6).mean() > 0.5  # most units are saturated
    S = int(got[6].sum())
    ups = [torch.randn(S, c, generator=gen) for c in (3, 3, 1, 3, 4)]
    sum((o * u.to(DEV)).sum() for o, u in zip(out[:5], ups)).backward()
    wd = orc.neural_gaussians_bwd(*_np_args(s), *[u.numpy() for u in ups], **kw)
    flat = [x for m in mlps for x in m]
    for i, (t, w) in enumerate(zip(flat, wd[4])):
        assert _rel(t.grad.cpu().numpy(), w) <= 1e-4, i


def test_no_anchor_and_nothing_selected():
    from gs_neural import neural_gaussians
    s = gs_scenes.make_anchor_scene(50, 10, 0)
    anchor, feat, offsets, scaling, campos, mlps = _to_dev(s, grad=True)
    out = neural_gaussians(anchor[:0], feat[:0], offsets[:0], scaling[:0], campos, *mlps)
    assert [tuple(o.shape) for o in out] == [(0, 3), (0, 3), (0, 1), (0, 3), (0, 4), (0, 1), (0,)]
    # an opacity bias far below zero switches every offset off
    off = [mlps[0][0], mlps[0][1], mlps[0][2], (mlps[0][3].detach() - 100.0).requires_grad_(True)]
    out = neural_gaussians(anchor, feat, offsets, scaling, campos, off, mlps[1], mlps[2])
    assert out[0].shape == (0, 3) and not bool(out[6].any())
    (out[0].sum() + out[4].sum()).backward()
    assert float(anchor.grad.abs().max()) == 0.0 and float(off[3].grad.abs().max()) == 0.0


def test_training_size_against_torch_statements():
    """200 k visible anchors, 10 offsets: forward and every gradient against the reference's statements run by
    torch on the device (float32; the selection can differ where an opacity is zero to rounding)."""
    from gs_neural import neural_gaussians
    N, k = 200_000, 10
    s = gs_scenes.make_anchor_scene(N, k, 21)
    a1 = _to_dev(s, grad=True)
    a2 = _to_dev(s, grad=True)
    out = neural_gaussians(*a1[:5], *a1[5])
    ref = gs_scenes.neural_gaussians_torch(*a2)
    assert float((out[5] - ref[5]).detach().abs().max()) <= 5e-6
    differ = out[6] != ref[6]
    assert int(differ.sum()) <= 20 and float(ref[5].view(-1)[differ].abs().max().item() if differ.any() else 0.0) <= 5e-6
    both = out[6] & ref[6]
    S = int(out[6].sum())
    assert 0.3 * N * k < S < 0.7 * N * k
    # compare on the offsets both selected; upstream gradients are given per slot so both sides use the same
    gen = torch.Generator(device=DEV).manual_seed(5)
    slot_up = [torch.randn(N * k, c, generator=gen, device=DEV) for c in (3, 3, 1, 3, 4)]
    for o_all, m in ((out, out[6]), (ref, ref[6])):
        keep, total = both[m], 0.0
        for o, u in zip(o_all[:5], slot_up):
            total = total + (o[keep] * u[m][keep]).sum()
        total.backward()
    for o, r in zip(out[:5], ref[:5]):
        assert float((o.detach()[both[out[6]]] - r.detach()[both[ref[6]]]).norm() / r.detach().norm()) <= 5e-6
    names = ("anchor", "feat", "offsets", "scaling")
    for name, x, y in zip(names, a1[:4], a2[:4]):
        assert float((x.grad - y.grad).norm() / y.grad.norm()) <= 1e-4, name
    for i, (x, y) in enumerate(zip([p for m in a1[5] for p in m], [p for m in a2[5] for p in m])):
        assert float((x.grad - y.grad).norm() / y.grad.norm()) <= 1e-3, i


def test_drop_in_signature():
    """generate_neural_gaussians(viewpoint_camera, pc, visible_mask, is_training) with a stand-in model object."""
    import types
    import torch.nn as nn
    from gs_neural import generate_neural_gaussians
    N, k = 500, 10
    s = gs_scenes.make_anchor_scene(N, k, 3)

    def seq(m, act):
        layers = [nn.Linear(35, 32), nn.ReLU(True), nn.Linear(32, m[2].shape[0])] + ([act] if act else [])
        q = nn.Sequential(*layers).to(DEV)
        with torch.no_grad():
            q[0].weight.copy_(m[0]); q[0].bias.copy_(m[1]); q[2].weight.copy_(m[2]); q[2].bias.copy_(m[3])
        return q

    pc = types.SimpleNamespace(
        use_feat_bank=False, appearance_dim=0, add_opacity_dist=False, add_color_dist=False, add_cov_dist=False,
        add_level=False, dist2level="round", n_offsets=k, get_anchor=s["anchor"].to(DEV),
        get_anchor_feat=s["feat"].to(DEV), _offset=s["offsets"].to(DEV), get_scaling=s["scaling"].to(DEV),
        get_opacity_mlp=seq(s["mlps"][0], nn.Tanh()), get_color_mlp=seq(s["mlps"][1], nn.Sigmoid()),
        get_cov_mlp=seq(s["mlps"][2], None))
    cam = types.SimpleNamespace(camera_center=s["campos"].to(DEV))
    vis = torch.rand(N, generator=torch.Generator().manual_seed(1)) < 0.6
    vis = vis.to(DEV)
    out = generate_neural_gaussians(cam, pc, vis, is_training=True)
    assert len(out) == 7 and len(generate_neural_gaussians(cam, pc, vis)) == 5
    ref = gs_scenes.neural_gaussians_torch(pc.get_anchor[vis], pc.get_anchor_feat[vis], pc._offset[vis],
                                           pc.get_scaling[vis], cam.camera_center,
                                           [tuple(x.to(DEV) for x in m) for m in s["mlps"]])
    assert torch.equal(out[6], ref[6])
    for o, r in zip(out[:6], ref[:6]):
        assert float((o.detach() - r.detach()).norm() / r.detach().norm()) <= 5e-6
    (out[1].sum() + out[3].sum()).backward()
    for q in (pc.get_color_mlp, pc.get_cov_mlp):
        for lin in (q[0], q[2]):
            assert bool(torch.isfinite(lin.weight.grad).all()) and float(lin.weight.grad.abs().max()) > 0.0
    assert float(pc.get_opacity_mlp[2].weight.grad.abs().max()) == 0.0
    # dist2level 'progressive': the model's ratio where transition_mask is set, 1 elsewhere (:844-848)
    pc.dist2level = "progressive"
    pc._prog_ratio = _prog(N, 1).to(DEV).clamp_min(0.01)
    pc.transition_mask = (torch.rand(N, generator=torch.Generator().manual_seed(2)) < 0.5).to(DEV)
    prog = pc._prog_ratio[vis].clone()
    prog[~pc.transition_mask[vis]] = 1.0
    out = generate_neural_gaussians(cam, pc, vis, is_training=True)
    ref = gs_scenes.neural_gaussians_torch(pc.get_anchor[vis], pc.get_anchor_feat[vis], pc._offset[vis],
                                           pc.get_scaling[vis], cam.camera_center,
                                           [tuple(x.to(DEV) for x in m) for m in s["mlps"]], prog)
    assert torch.equal(out[6], ref[6])
    for o, r in zip(out[:6], ref[:6]):
        assert float((o.detach() - r.detach()).norm() / r.detach().norm()) <= 5e-6
    # and without a visibility mask
    out = generate_neural_gaussians(cam, pc, None, is_training=True)
    full = torch.where(pc.transition_mask[:, None], pc._prog_ratio, torch.ones_like(pc._prog_ratio))
    ref = gs_scenes.neural_gaussians_torch(pc.get_anchor, pc.get_anchor_feat, pc._offset, pc.get_scaling,
                                           cam.camera_center, [tuple(x.to(DEV) for x in m) for m in s["mlps"]], full)
    assert torch.equal(out[6], ref[6])
    assert float((out[5] - ref[5]).norm() / ref[5].norm()) <= 5e-6


def test_drop_in_with_distance_and_level_inputs():
    """add_opacity_dist, add_cov_dist, add_level, the feature bank with the level and the appearance embedding behind
    the level column, against the reference's statements run by torch (gaussian_renderer/__init__.py:800-896)."""
    import types
    import torch.nn as nn
    from gs_neural import generate_neural_gaussians
    N, k, A = 300, 10, 16
    s = gs_scenes.make_anchor_scene(N, k, 17)
    torch.manual_seed(5)
    mlp_op = nn.Sequential(nn.Linear(37, 32), nn.ReLU(True), nn.Linear(32, k), nn.Tanh()).to(DEV)
    mlp_cov = nn.Sequential(nn.Linear(37, 32), nn.ReLU(True), nn.Linear(32, 7 * k)).to(DEV)
    mlp_col = nn.Sequential(nn.Linear(36 + A, 32), nn.ReLU(True), nn.Linear(32, 3 * k), nn.Sigmoid()).to(DEV)
    bank = nn.Sequential(nn.Linear(4, 32), nn.ReLU(True), nn.Linear(32, 3), nn.Softmax(dim=1)).to(DEV)
    emb = nn.Embedding(5, A).to(DEV)
    leaf = lambda t: t.to(DEV).requires_grad_(True)
    pc = types.SimpleNamespace(
        use_feat_bank=True, appearance_dim=A, add_opacity_dist=True, add_color_dist=False, add_cov_dist=True,
        add_level=True, dist2level="round", n_offsets=k, get_anchor=leaf(s["anchor"]),
        get_anchor_feat=leaf(s["feat"]), _offset=leaf(s["offsets"]), get_scaling=leaf(s["scaling"]),
        get_level=s["level"].to(DEV), get_opacity_mlp=mlp_op, get_color_mlp=mlp_col, get_cov_mlp=mlp_cov,
        get_featurebank_mlp=bank, get_appearance=emb)
    cam = types.SimpleNamespace(camera_center=s["campos"].to(DEV), uid=2)
    vis = (torch.rand(N, generator=torch.Generator().manual_seed(3)) < 0.7).to(DEV)

    def reference():
        anchor, feat, level = pc.get_anchor[vis], pc.get_anchor_feat[vis], pc.get_level[vis]
        grid_offsets, grid_scaling = pc._offset[vis], pc.get_scaling[vis]
        ob_view = anchor - cam.camera_center
        ob_dist = ob_view.norm(dim=1, keepdim=True)
        ob_view = ob_view / ob_dist
        bank_weight = bank(torch.cat([ob_view, level], dim=1)).unsqueeze(dim=1)
        feat = feat.unsqueeze(dim=-1)
        feat = feat[:, ::4, :1].repeat([1, 4, 1]) * bank_weight[:, :, :1] + \
            feat[:, ::2, :1].repeat([1, 2, 1]) * bank_weight[:, :, 1:2] + feat[:, ::1, :1] * bank_weight[:, :, 2:]
        feat = feat.squeeze(dim=-1)
        cat_local_view = torch.cat([feat, ob_view, ob_dist, level], dim=1)
        cat_local_view_wodist = torch.cat([feat, ob_view, level], dim=1)
        camera_indicies = torch.ones_like(cat_local_view[:, 0], dtype=torch.long) * cam.uid
        appearance = emb(camera_indicies)
        neural_opacity = mlp_op(cat_local_view).reshape([-1, 1])
        mask = (neural_opacity > 0.0).view(-1)
        opacity = neural_opacity[mask]
        color = mlp_col(torch.cat([cat_local_view_wodist, appearance], dim=1)).reshape([anchor.shape[0] * k, 3])
        scale_rot = mlp_cov(cat_local_view).reshape([anchor.shape[0] * k, 7])
        offsets = grid_offsets.view([-1, 3])
        cat = torch.cat([grid_scaling, anchor], dim=-1).repeat_interleave(k, dim=0)
        masked = torch.cat([cat, color, scale_rot, offsets], dim=-1)[mask]
        scaling_repeat, repeat_anchor, color, scale_rot, offsets = masked.split([6, 3, 3, 7, 3], dim=-1)
        scaling = scaling_repeat[:, 3:] * torch.sigmoid(scale_rot[:, :3])
        rot = torch.nn.functional.normalize(scale_rot[:, 3:7])
        xyz = repeat_anchor + offsets * scaling_repeat[:, :3]
        return xyz, color, opacity, scaling, rot, neural_opacity, mask

    params = [pc.get_anchor, pc.get_anchor_feat, pc._offset, pc.get_scaling, emb.weight] + \
        [p for m in (mlp_op, mlp_col, mlp_cov, bank) for p in m.parameters()]
    gen = torch.Generator().manual_seed(9)
    results = []
    for fn in (reference, lambda: generate_neural_gaussians(cam, pc, vis, is_training=True)):
        for p in params:
            p.grad = None
        out = fn()
        if not results:
            ups = [torch.randn(out[0].shape[0], c, generator=gen).to(DEV) for c in (3, 3, 1, 3, 4)]
        sum((o * u).sum() for o, u in zip(out[:5], ups)).backward()
        results.append(([o.detach().clone() for o in out], [p.grad.detach().clone() for p in params]))
    (ref_out, ref_grad), (got_out, got_grad) = results
    assert torch.equal(ref_out[6], got_out[6])
    for r, g in zip(ref_out[:6], got_out[:6]):
        assert float((g - r).norm() / r.norm()) <= 1e-5
    for i, (r, g) in enumerate(zip(ref_grad, got_grad)):
        assert float((g - r).norm() / r.norm()) <= 2e-4, i


def test_drop_in_with_appearance_embedding_and_feature_bank():
    """appearance_dim > 0 and use_feat_bank, against the reference's statements for them
    (gaussian_renderer/__init__.py:809-836, :866-870) run by torch."""
    import types
    import torch.nn as nn
    from gs_neural import generate_neural_gaussians
    N, k, A = 400, 10, 32
    s = gs_scenes.make_anchor_scene(N, k, 13)
    torch.manual_seed(4)
    mlp_op = nn.Sequential(nn.Linear(35, 32), nn.ReLU(True), nn.Linear(32, k), nn.Tanh()).to(DEV)
    mlp_cov = nn.Sequential(nn.Linear(35, 32), nn.ReLU(True), nn.Linear(32, 7 * k)).to(DEV)
    mlp_col = nn.Sequential(nn.Linear(35 + A, 32), nn.ReLU(True), nn.Linear(32, 3 * k), nn.Sigmoid()).to(DEV)
    bank = nn.Sequential(nn.Linear(3, 32), nn.ReLU(True), nn.Linear(32, 3), nn.Softmax(dim=1)).to(DEV)
    emb = nn.Embedding(7, A).to(DEV)
    leaf = lambda t: t.to(DEV).requires_grad_(True)
    pc = types.SimpleNamespace(
        use_feat_bank=True, appearance_dim=A, add_opacity_dist=False, add_color_dist=False, add_cov_dist=False,
        add_level=False, dist2level="round", n_offsets=k, get_anchor=leaf(s["anchor"]),
        get_anchor_feat=leaf(s["feat"]), _offset=leaf(s["offsets"]), get_scaling=leaf(s["scaling"]),
        get_opacity_mlp=mlp_op, get_color_mlp=mlp_col, get_cov_mlp=mlp_cov, get_featurebank_mlp=bank,
        get_appearance=emb)
    cam = types.SimpleNamespace(camera_center=s["campos"].to(DEV), uid=3)
    vis = (torch.rand(N, generator=torch.Generator().manual_seed(2)) < 0.7).to(DEV)

    def reference():
        anchor, feat = pc.get_anchor[vis], pc.get_anchor_feat[vis]
        grid_offsets, grid_scaling = pc._offset[vis], pc.get_scaling[vis]
        ob_view = anchor - cam.camera_center
        ob_dist = ob_view.norm(dim=1, keepdim=True)
        ob_view = ob_view / ob_dist
        bank_weight = bank(ob_view).unsqueeze(dim=1)
        feat = feat.unsqueeze(dim=-1)
        feat = feat[:, ::4, :1].repeat([1, 4, 1]) * bank_weight[:, :, :1] + \
            feat[:, ::2, :1].repeat([1, 2, 1]) * bank_weight[:, :, 1:2] + feat[:, ::1, :1] * bank_weight[:, :, 2:]
        feat = feat.squeeze(dim=-1)
        x = torch.cat([feat, ob_view], dim=1)
        camera_indicies = torch.ones_like(x[:, 0], dtype=torch.long) * cam.uid
        appearance = emb(camera_indicies)
        neural_opacity = mlp_op(x).reshape([-1, 1])
        mask = (neural_opacity > 0.0).view(-1)
        opacity = neural_opacity[mask]
        color = mlp_col(torch.cat([x, appearance], dim=1)).reshape([anchor.shape[0] * k, 3])
        scale_rot = mlp_cov(x).reshape([anchor.shape[0] * k, 7])
        offsets = grid_offsets.view([-1, 3])
        cat = torch.cat([grid_scaling, anchor], dim=-1).repeat_interleave(k, dim=0)
        masked = torch.cat([cat, color, scale_rot, offsets], dim=-1)[mask]
        scaling_repeat, repeat_anchor, color, scale_rot, offsets = masked.split([6, 3, 3, 7, 3], dim=-1)
        scaling = scaling_repeat[:, 3:] * torch.sigmoid(scale_rot[:, :3])
        rot = torch.nn.functional.normalize(scale_rot[:, 3:7])
        xyz = repeat_anchor + offsets * scaling_repeat[:, :3]
        return xyz, color, opacity, scaling, rot, neural_opacity, mask

    params = [pc.get_anchor, pc.get_anchor_feat, pc._offset, pc.get_scaling, emb.weight] + \
        [p for m in (mlp_op, mlp_col, mlp_cov, bank) for p in m.parameters()]
    ups = None
    grads = []
    for fn in (lambda: generate_neural_gaussians(cam, pc, vis, is_training=True), reference):
        for p in params:
            p.grad = None
        out = fn()
        if ups is None:
            ups = [torch.randn_like(o) for o in out[:5]]
            first = out
        else:
            assert torch.equal(out[6], first[6])
            for o, r in zip(first[:6], out[:6]):
                assert float((o.detach() - r.detach()).norm() / r.detach().norm()) <= 5e-6
        torch.autograd.backward(list(out[:5]), ups)
        grads.append([p.grad.clone() for p in params])
    for i, (a, b) in enumerate(zip(*grads)):
        assert float((a - b).norm()) <= 2e-4 * float(b.norm()) + 1e-12, i
