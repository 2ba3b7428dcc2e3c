"""Fused multi-tensor Adam on the GPU: through the C ABI against the numpy oracle, and the optimizer class
against torch.optim.Adam stepping the same parameters."""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


def test_adam_c_abi_matches_oracle(orc):
    import gsrast_native as gn
    gen = torch.Generator().manual_seed(3)
    # sizes around the 4096-element workgroup chunk, a misaligned view, an empty tensor, 30 tensors (> one launch)
    sizes = [1, 3, 4095, 4096, 4097, 100_003, 0, 1_000_000] + [17 + 13 * i for i in range(22)]
    store = [torch.randn(n + 1, generator=gen).to(DEV) for n in sizes]
    before5 = float(store[5][0])
    p = [s[1:] if i == 5 else s[:n] for i, (s, n) in enumerate(zip(store, sizes))]  # tensor 5 starts 4 bytes off
    g = [(torch.randn(n, generator=gen) * 0.1).to(DEV) for n in sizes]
    m = [(torch.randn(n, generator=gen) * 0.01).to(DEV) for n in sizes]
    v = [(torch.rand(n, generator=gen) * 1e-4).to(DEV) for n in sizes]
    lrs = [10.0 ** -(2 + i % 4) for i in range(len(sizes))]
    steps = [1 + (i * 7) % 50 for i in range(len(sizes))]
    ref = [orc.adam_step(a.cpu().numpy(), b.cpu().numpy(), c.cpu().numpy(), d.cpu().numpy(), lr, st, grad_scale=0.5)
           for a, b, c, d, lr, st in zip(p, g, m, v, lrs, steps)]
    n = len(sizes)
    vp = C.c_void_p * n
    rc = gn.lib.gs_adam_step(n, vp(*[t.data_ptr() for t in p]), vp(*[t.data_ptr() for t in g]),
                             vp(*[t.data_ptr() for t in m]), vp(*[t.data_ptr() for t in v]),
                             (C.c_longlong * n)(*sizes), (C.c_double * n)(*lrs), (C.c_int * n)(*steps), 0.9, 0.999,
                             1e-15, 0.5, C.c_void_p(torch.cuda.current_stream().cuda_stream))
    gn.check(rc, "gs_adam_step")
    torch.cuda.synchronize()
    assert float(store[5][0]) == before5  # the element in front of the misaligned view is untouched
    for i, (rp, rm, rv) in enumerate(ref):
        if sizes[i] == 0:
            continue
        # same operations in the same order: at most a last-bit difference (sqrt and division are IEEE on both)
        assert np.abs(m[i].cpu().numpy() - rm).max() <= 1e-7 * np.abs(rm).max()
        assert np.abs(v[i].cpu().numpy() - rv).max() <= 1e-7 * np.abs(rv).max()
        assert np.abs(p[i].cpu().numpy() - rp).max() <= 1e-6 * max(1.0, np.abs(rp).max())
    # a step number of 0 is refused (steps count from 1)
    one = lambda t: (C.c_void_p * 1)(t.data_ptr())
    with pytest.raises(RuntimeError, match="step numbers"):
        gn.check(gn.lib.gs_adam_step(1, one(p[0]), one(g[0]), one(m[0]), one(v[0]), (C.c_longlong * 1)(1),
                                     (C.c_double * 1)(1e-3), (C.c_int * 1)(0), 0.9, 0.999, 1e-15, 1.0, None),
                 "gs_adam_step")


def test_fused_adam_tracks_torch_adam():
    from gs_optim import FusedAdam
    gen = torch.Generator().manual_seed(9)
    shapes = [(50_000, 3), (50_000, 10, 3), (50_000, 1), (32, 35), (32,)]
    lrs = [1.6e-4, 7.5e-3, 0.02, 2e-3, 2e-3]
    init = [torch.randn(s, generator=gen) for s in shapes]
    mine = [t.clone().to(DEV).requires_grad_(True) for t in init]
    theirs = [t.clone().to(DEV).requires_grad_(True) for t in init]
    groups = lambda ps: [{"params": [p], "lr": lr, "name": f"g{i}"} for i, (p, lr) in enumerate(zip(ps, lrs))]
    a = FusedAdam(groups(mine), lr=0.0, eps=1e-15, grad_scale=0.25)
    b = torch.optim.Adam(groups(theirs), lr=0.0, eps=1e-15)
    for it in range(8):
        for i, (x, y) in enumerate(zip(mine, theirs)):
            if it == 3 and i == 2:
                x.grad = None  # a parameter without a gradient is skipped and keeps its step count
                y.grad = None
                continue
            gr = (torch.randn(x.shape, generator=gen) * 10.0 ** (it % 3 - 1)).to(DEV)
            x.grad = gr.clone()
            y.grad = gr * 0.25  # the reference divides the gradients by the batch size before stepping
        a.step()
        b.step()
    for x, y, t0 in zip(mine, theirs, init):
        assert _rel((x.detach().cpu() - t0).numpy(), (y.detach().cpu() - t0).numpy()) <= 1e-5
        sa, sb = a.state[x], b.state[y]
        assert int(sa["step"]) == int(sb["step"])
        assert _rel(sa["exp_avg"].cpu().numpy(), sb["exp_avg"].cpu().numpy()) <= 1e-6
        assert _rel(sa["exp_avg_sq"].cpu().numpy(), sb["exp_avg_sq"].cpu().numpy()) <= 1e-6
    # state layout is torch.optim.Adam's: a state dict moves between the two
    b2 = torch.optim.Adam(groups(theirs), lr=0.0, eps=1e-15)
    b2.load_state_dict(a.state_dict())
    assert int(b2.state[theirs[0]]["step"]) == 8
    with pytest.raises(RuntimeError):
        c = FusedAdam([torch.zeros(3, requires_grad=True)], lr=1e-3)
        c.param_groups[0]["params"][0].grad = torch.ones(3)
        c.step()
