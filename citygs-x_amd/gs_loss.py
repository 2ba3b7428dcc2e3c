"""The per-pixel loss maps of the reference, utils/loss_utils.py:88-132, as one fused call each way into
libgsrast.so.  `pixelwise_l1_with_mask` and `pixelwise_ssim_with_mask` keep the reference's names and
arguments; `pixelwise_l1_ssim_with_mask` returns both maps from a single pass, which is what
gaussian_renderer/loss_distribution.py:267-279 needs."""
import ctypes as C

import torch

import gsrast_native as _n


def _p(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _img(t, name):
    if t.dim() != 3:
        raise RuntimeError(f"{name} must be (channels, height, width)")
    if t.dtype != torch.float32:
        raise TypeError(f"{name} must be float32, got {t.dtype}")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a GPU tensor: there is no CPU path")
    return t.contiguous()


class _L1SsimMaps(torch.autograd.Function):
    @staticmethod
    def forward(ctx, img1, img2, pixel_mask):
        a, b = _img(img1, "img1"), _img(img2, "img2")
        if a.shape != b.shape:
            raise RuntimeError("img1 and img2 must have the same shape")
        Cn, H, W = a.shape
        m = None
        if pixel_mask is not None:
            if pixel_mask.shape != (H, W) or pixel_mask.dtype not in (torch.bool, torch.uint8) or not pixel_mask.is_cuda:
                raise RuntimeError("pixel_mask must be a (height, width) bool GPU tensor")
            m = pixel_mask.contiguous().view(torch.uint8)
        l1, ss = torch.empty_like(a), torch.empty_like(a)
        need = ctx.needs_input_grad[0]
        d = [torch.empty_like(a) for _ in range(3)] if need else [None, None, None]
        stream = C.c_void_p(torch.cuda.current_stream(a.device).cuda_stream)
        _n.check(_n.lib.gs_ssim_l1_forward(Cn, H, W, _p(a), _p(b), _p(m), _p(l1), _p(ss), _p(d[0]), _p(d[1]), _p(d[2]),
                                           stream), "pixelwise_l1_ssim_with_mask")
        if need:
            ctx.save_for_backward(a, b, m, *d)
        ctx.set_materialize_grads(False)
        return l1, ss

    @staticmethod
    def backward(ctx, g_l1, g_ssim):
        a, b, m, d_mu, d_xx, d_xy = ctx.saved_tensors
        Cn, H, W = a.shape
        if g_l1 is None and g_ssim is None:
            return torch.zeros_like(a), None, None
        g1 = None if g_l1 is None else _img(g_l1, "grad of l1 map")
        g2 = None if g_ssim is None else _img(g_ssim, "grad of ssim map")
        out = torch.empty_like(a)
        stream = C.c_void_p(torch.cuda.current_stream(a.device).cuda_stream)
        _n.check(_n.lib.gs_ssim_l1_backward(Cn, H, W, _p(a), _p(b), _p(m), _p(g1), _p(g2), _p(d_mu), _p(d_xx),
                                            _p(d_xy), _p(out), stream), "pixelwise_l1_ssim_with_mask backward")
        return out, None, None


def pixelwise_l1_ssim_with_mask(img1, img2, pixel_mask=None):
    """(|img1 - img2| * mask, SSIM(img1, img2) * mask), both (3, H, W); differentiable in img1 (img2 is the
    ground truth and gets no gradient)."""
    return _L1SsimMaps.apply(img1, img2, pixel_mask)


def pixelwise_l1_with_mask(img1, img2, pixel_mask):
    """utils/loss_utils.py:88-94."""
    return _L1SsimMaps.apply(img1, img2, pixel_mask)[0]


def pixelwise_ssim_with_mask(img1, img2, pixel_mask):
    """utils/loss_utils.py:97-132."""
    return _L1SsimMaps.apply(img1, img2, pixel_mask)[1]
