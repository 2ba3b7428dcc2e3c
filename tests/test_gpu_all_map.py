"""The fused per-Gaussian geometry-channel op (gaussian_renderer/__init__.py:1501-1518) on the GPU:
through the C ABI against the CPU oracle, and through the autograd op against the torch lines it replaces."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def H():
    import gpu_harness
    return gpu_harness


@pytest.mark.parametrize("cfg,P", [(0, 50_000), (1, 200_003), (3, 100_000)])
def test_all_map_c_abi_matches_oracle(H, orc, cfg, P):
    import gs_scenes
    g, cams = gs_scenes.make_scene(cfg, P=P, n_views=1)
    cam = cams[0]
    lib, gn = H.lib, H.gn
    rots = g["rotations"] * torch.linspace(0.5, 2.0, P)[:, None]  # unnormalised, like raw parameters
    m, s, q = H.dev(g["means3D"]), H.dev(g["scales"]), H.dev(rots)
    V, cp = H.dev(cam.world_view_transform), H.dev(cam.camera_center)
    out = torch.full((P, 5), float("nan"), device=DEV)
    gn.check(lib.gs_all_map_forward(P, H.ptr(m), H.ptr(s), H.ptr(q), H.ptr(V), H.ptr(cp), H.ptr(out), H.stream()),
             "gs_all_map_forward")
    ref = orc.all_map_fwd(g["means3D"].numpy(), g["scales"].numpy(), rots.numpy(), cam.world_view_transform.numpy(),
                          cam.camera_center.numpy())
    got = out.cpu().numpy()
    # same operations in the same order on both sides: allow a last-bit difference, no more
    assert np.abs(got - ref).max() <= 1e-6 * max(1.0, np.abs(ref).max())
    go = torch.randn(P, 5, generator=torch.Generator().manual_seed(cfg))
    dm = torch.full((P, 3), float("nan"), device=DEV)
    dq = torch.full((P, 4), float("nan"), device=DEV)
    gd = H.dev(go)
    gn.check(lib.gs_all_map_backward(P, H.ptr(m), H.ptr(s), H.ptr(q), H.ptr(V), H.ptr(cp), H.ptr(gd), H.ptr(dm),
                                     H.ptr(dq), H.stream()), "gs_all_map_backward")
    rm, rq = orc.all_map_bwd(g["means3D"].numpy(), g["scales"].numpy(), rots.numpy(), cam.world_view_transform.numpy(),
                             cam.camera_center.numpy(), go.numpy())
    assert H.rel_l2(dm.cpu().numpy(), rm) <= 1e-6
    assert H.rel_l2(dq.cpu().numpy(), rq) <= 1e-6


def test_all_map_op_replaces_the_torch_lines(H):
    import gs_scenes
    from diff_gaussian_rasterization import build_all_map
    g, cams = gs_scenes.make_scene(1, P=120_000, n_views=1)
    cam = cams[0]
    V, cp = cam.world_view_transform.to(DEV), cam.camera_center.to(DEV)
    leaf = {k: g[k].to(DEV).requires_grad_(True) for k in ("means3D", "scales", "rotations")}
    ours = build_all_map(leaf["means3D"], leaf["scales"], leaf["rotations"], V, cp)
    go = torch.randn(ours.shape, generator=torch.Generator().manual_seed(4)).to(DEV)
    (ours * go).sum().backward()
    got = {k: (None if v.grad is None else v.grad.clone()) for k, v in leaf.items()}
    for v in leaf.values():
        v.grad = None
    theirs = gs_scenes.build_all_map(leaf["means3D"], leaf["scales"], leaf["rotations"], cam)
    (theirs * go).sum().backward()
    # a normal whose dot product with the view direction is at rounding level may flip either way
    nrm = theirs[:, :3].detach()
    stable = (nrm - ours[:, :3].detach()).abs().amax(1) < 1.0
    assert float(stable.float().mean()) > 0.9999
    assert float((ours.detach() - theirs.detach())[stable].abs().max()) <= 1e-4
    assert got["scales"] is None
    for k in ("means3D", "rotations"):
        a, b = got[k][stable].double(), leaf[k].grad[stable].double()
        assert float((a - b).norm() / b.norm()) <= 1e-5


def test_all_map_empty_and_errors():
    from diff_gaussian_rasterization import build_all_map
    z = torch.zeros(0, 3, device=DEV)
    out = build_all_map(z, z, torch.zeros(0, 4, device=DEV), torch.eye(4, device=DEV), torch.zeros(3, device=DEV))
    assert out.shape == (0, 5)
    with pytest.raises(RuntimeError):
        build_all_map(torch.zeros(4, 3), torch.zeros(4, 3), torch.zeros(4, 4), torch.eye(4), torch.zeros(3))
