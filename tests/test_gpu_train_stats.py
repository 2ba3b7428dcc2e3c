"""Densification statistics (GaussianModel.training_statis, scene/gaussian_model.py:1181-1205) on the GPU:
the fused call against the CPU oracle and against torch's own mask indexing on the device."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _case(A, k, seed, p_vis, p_sel, p_flt):
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


@pytest.mark.parametrize("A,k,seed,p", [(5000, 10, 0, (0.6, 0.7, 0.8)), (4097, 5, 1, (1.0, 1.0, 1.0)),
                                        (3000, 10, 2, (0.02, 0.3, 0.5)), (2048, 1, 3, (0.5, 0.5, 0.0)),
                                        (1000, 10, 4, (0.0, 0.5, 0.5))])
def test_training_stats_matches_oracle(orc, A, k, seed, p):
    import gs_densify
    vis, sel, flt, grad, opacity, acc = _case(A, k, seed, *p)
    ref = orc.training_stats(acc[0].numpy(), acc[1].numpy(), acc[2].numpy(), acc[3].numpy(), k, grad.numpy(),
                             opacity.numpy(), flt.numpy(), sel.numpy(), vis.numpy())
    d = [t.to(DEV) for t in acc]
    gs_densify.training_statis(d[0], d[1], d[2], d[3], k, grad.to(DEV), opacity.to(DEV), flt.to(DEV), sel.to(DEV),
                               vis.to(DEV))
    for got, want in zip(d, ref):
        # same additions in the same order (one per slot and call): identical up to the last bit of sqrt's input
        assert np.abs(got.cpu().numpy().ravel() - want).max() <= 1e-6 * max(1.0, np.abs(want).max())


def test_training_stats_full_size_against_mask_indexing():
    """1 M anchors x 10 offsets, checked against the torch statements it replaces, run on the device."""
    import gs_densify
    A, k = 1_000_000, 10
    gen = torch.Generator(device=DEV).manual_seed(5)
    vis = torch.rand(A, generator=gen, device=DEV) < 0.4
    V = int(vis.sum())
    sel = torch.rand(V * k, generator=gen, device=DEV) < 0.6
    S = int(sel.sum())
    flt = torch.rand(S, generator=gen, device=DEV) < 0.9
    grad = torch.randn(S, 3, generator=gen, device=DEV)
    opacity = torch.randn(V * k, 1, generator=gen, device=DEV)
    acc = [torch.zeros(A, 1, device=DEV), torch.zeros(A, 1, device=DEV), torch.zeros(A * k, 1, device=DEV),
           torch.zeros(A * k, 1, device=DEV)]
    mine = [t.clone() for t in acc]
    for _ in range(2):  # twice: accumulation, not assignment
        gs_densify.training_statis(mine[0], mine[1], mine[2], mine[3], k, grad, opacity, flt, sel, vis)
        temp = opacity.clone().view(-1)
        temp[temp < 0] = 0
        acc[0][vis] += temp.view(-1, k).sum(dim=1, keepdim=True)
        acc[1][vis] += 1
        vis_rep = vis.unsqueeze(1).repeat(1, k).view(-1)
        combined = torch.zeros(A * k, dtype=torch.bool, device=DEV)
        combined[vis_rep] = sel
        temp_mask = combined.clone()
        combined[temp_mask] = flt
        acc[2][combined] += torch.norm(grad[flt, :2], dim=-1, keepdim=True)
        acc[3][combined] += 1
    assert torch.equal(mine[1], acc[1]) and torch.equal(mine[3], acc[3])
    assert float((mine[0] - acc[0]).abs().max()) <= 1e-5
    assert float((mine[2] - acc[2]).abs().max()) <= 1e-5
    assert int(mine[3].sum()) == 2 * int(flt.sum())


def test_training_stats_rejects_inconsistent_inputs():
    import gs_densify
    z = lambda *s: torch.zeros(*s, device=DEV)
    with pytest.raises(RuntimeError):
        gs_densify.training_statis(z(4, 1), z(4, 1), z(8, 1), z(8, 1), 2, z(3, 3), z(5, 1),
                                   torch.ones(3, dtype=torch.bool, device=DEV),
                                   torch.ones(5, dtype=torch.bool, device=DEV),
                                   torch.ones(4, dtype=torch.bool, device=DEV))
    with pytest.raises(RuntimeError):
        gs_densify.training_statis(torch.zeros(4, 1), torch.zeros(4, 1), torch.zeros(8, 1), torch.zeros(8, 1), 2,
                                   torch.zeros(0, 3), torch.zeros(0, 1), torch.zeros(0, dtype=torch.bool),
                                   torch.zeros(0, dtype=torch.bool), torch.zeros(4, dtype=torch.bool))


def test_update_max_radii_matches_torch_statement():
    import gs_densify
    gen = torch.Generator().manual_seed(3)
    n = 100_003
    m = torch.rand(n, generator=gen) * 40
    radii = torch.randint(0, 80, (n,), generator=gen, dtype=torch.int32)
    vis = torch.rand(n, generator=gen) < 0.4
    want = m.clone()
    want[vis] = torch.max(want[vis], radii[vis].float())
    got = gs_densify.update_max_radii(m.to(DEV), radii.to(DEV), vis.to(DEV)).cpu()
    assert torch.equal(got, want)
    assert torch.equal(got[~vis], m[~vis])
