"""Drop-in for the optimizer of the reference, torch.optim.Adam(l, lr=0.0, eps=1e-15) over named parameter
groups with their own learning rates (scene/gaussian_model.py:561-574): same constructor, param_groups and
per-parameter state ("step", "exp_avg", "exp_avg_sq"), so the reference's optimizer surgery when anchors are
added or pruned (scene/gaussian_model.py:1133-1177, 1208-1243) and its checkpoints keep working.  step()
updates every parameter that has a gradient in one kernel launch of libgsrast.so."""
import ctypes as C

import torch

import gsrast_native as _n


class FusedAdam(torch.optim.Optimizer):
    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, grad_scale=1.0):
        if lr < 0.0 or eps < 0.0 or not (0.0 <= betas[0] < 1.0) or not (0.0 <= betas[1] < 1.0):
            raise ValueError("invalid Adam hyper-parameter")
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps))
        # multiplies every gradient inside the update (the reference divides param.grad by the batch size
        # just before stepping, train_internal.py:407-410)
        self.grad_scale = float(grad_scale)

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        # one launch per (betas, eps, device) combination; the reference has a single one
        batches = {}
        for group in self.param_groups:
            for p in group["params"]:
                if p.grad is None:
                    continue
                if p.grad.is_sparse:
                    raise RuntimeError("FusedAdam does not support sparse gradients")
                if p.dtype != torch.float32 or not p.is_cuda:
                    raise RuntimeError("FusedAdam updates float32 GPU parameters only: there is no CPU path")
                if not p.is_contiguous():
                    raise RuntimeError("FusedAdam needs contiguous parameters")
                state = self.state[p]
                if len(state) == 0:
                    state["step"] = torch.tensor(0.0)
                    state["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                    state["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                state["step"] = state["step"] + 1 if torch.is_tensor(state["step"]) else state["step"] + 1
                key = (group["betas"][0], group["betas"][1], group["eps"], p.device)
                batches.setdefault(key, []).append((p, p.grad.contiguous(), state, group["lr"]))
        for (b1, b2, eps, dev), items in batches.items():
            n = len(items)
            ptr_t = C.c_void_p * n
            params = ptr_t(*[p.data_ptr() for p, _, _, _ in items])
            grads = ptr_t(*[g.data_ptr() for _, g, _, _ in items])
            m = ptr_t(*[s["exp_avg"].data_ptr() for _, _, s, _ in items])
            v = ptr_t(*[s["exp_avg_sq"].data_ptr() for _, _, s, _ in items])
            sizes = (C.c_longlong * n)(*[p.numel() for p, _, _, _ in items])
            lrs = (C.c_double * n)(*[float(lr) for _, _, _, lr in items])
            steps = (C.c_int * n)(*[int(s["step"]) for _, _, s, _ in items])
            stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
            with torch.cuda.device(dev):
                _n.check(_n.lib.gs_adam_step(n, params, grads, m, v, sizes, lrs, steps, float(b1), float(b2),
                                             float(eps), self.grad_scale, stream), "FusedAdam.step")
        return loss
