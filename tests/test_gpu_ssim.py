"""Fused masked L1 + SSIM maps (utils/loss_utils.py:88-132) on the GPU: against the CPU oracle at sizes it
finishes quickly, and at the training resolution against torch's own conv2d formulation on the device."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _images(Cn, H, W, seed):
    gen = torch.Generator().manual_seed(seed)
    a = torch.rand(Cn, H, W, generator=gen)
    b = (a + 0.15 * torch.randn(Cn, H, W, generator=gen)).clamp(0, 1)
    mask = torch.rand(H, W, generator=gen) < 0.8
    return a, b, mask


@pytest.mark.parametrize("Cn,H,W,use_mask", [(3, 64, 96, True), (3, 37, 53, True), (1, 16, 16, False), (3, 5, 7, True),
                                             (2, 130, 17, False)])
def test_maps_and_gradient_match_oracle(orc, Cn, H, W, use_mask):
    from gs_loss import pixelwise_l1_ssim_with_mask
    a, b, mask = _images(Cn, H, W, seed=H * W)
    m = mask if use_mask else None
    x = a.to(DEV).requires_grad_(True)
    l1, ss = pixelwise_l1_ssim_with_mask(x, b.to(DEV), None if m is None else m.to(DEV))
    rl1, rss = orc.ssim_l1_fwd(a.numpy(), b.numpy(), None if m is None else m.numpy())
    assert np.abs(l1.detach().cpu().numpy() - rl1).max() <= 1e-7
    # same window and formula; the kernel sums the window as two 1-D passes, the oracle as one 2-D sum
    assert np.abs(ss.detach().cpu().numpy() - rss).max() <= 1e-5
    gen = torch.Generator().manual_seed(7)
    g1, g2 = torch.randn(Cn, H, W, generator=gen), torch.randn(Cn, H, W, generator=gen)
    ((l1 * g1.to(DEV)).sum() + (ss * g2.to(DEV)).sum()).backward()
    rd = orc.ssim_l1_bwd(a.numpy(), b.numpy(), None if m is None else m.numpy(), g1.numpy(), g2.numpy())
    got = x.grad.cpu().numpy()
    assert np.linalg.norm(got - rd) / np.linalg.norm(rd) <= 1e-5


def test_training_resolution_against_torch_statements():
    """1152x864x3, the loss exactly as loss_distribution.py:267-279 forms it, both ways on the device."""
    import torch.nn.functional as F
    import gs_loss
    Cn, H, W = 3, 864, 1152
    a, b, mask = _images(Cn, H, W, seed=3)
    a, b, mask = a.to(DEV), b.to(DEV), mask.to(DEV)

    def reference(img1, img2, pixel_mask):
        import math
        g = torch.Tensor([math.exp(-((x - 5) ** 2) / float(2 * 1.5 ** 2)) for x in range(11)])
        g = (g / g.sum()).unsqueeze(1)
        window = g.mm(g.t()).float().unsqueeze(0).unsqueeze(0).expand(Cn, 1, 11, 11).contiguous().to(DEV)
        mu1 = F.conv2d(img1, window, padding=5, groups=Cn)
        mu2 = F.conv2d(img2, window, padding=5, groups=Cn)
        mu1_sq, mu2_sq, mu1_mu2 = mu1.pow(2), mu2.pow(2), mu1 * mu2
        s1 = F.conv2d(img1 * img1, window, padding=5, groups=Cn) - mu1_sq
        s2 = F.conv2d(img2 * img2, window, padding=5, groups=Cn) - mu2_sq
        s12 = F.conv2d(img1 * img2, window, padding=5, groups=Cn) - mu1_mu2
        m = ((2 * mu1_mu2 + 0.01 ** 2) * (2 * s12 + 0.03 ** 2)) / ((mu1_sq + mu2_sq + 0.01 ** 2) * (s1 + s2 + 0.03 ** 2))
        return torch.abs(img1 - img2) * pixel_mask.unsqueeze(0), m * pixel_mask.unsqueeze(0)

    x1 = a.clone().requires_grad_(True)
    l1, ss = gs_loss.pixelwise_l1_ssim_with_mask(x1, b, mask)
    loss1 = (0.8 * l1.sum() + 0.2 * (mask.sum() * Cn - ss.sum())) / (H * W * Cn)
    loss1.backward()
    x2 = a.clone().requires_grad_(True)
    rl1, rss = reference(x2, b, mask)
    loss2 = (0.8 * rl1.sum() + 0.2 * (mask.sum() * Cn - rss.sum())) / (H * W * Cn)
    loss2.backward()
    assert torch.equal(l1, rl1)
    assert float((ss.detach() - rss.detach()).abs().max()) <= 2e-5
    assert abs(float(loss1.detach()) - float(loss2.detach())) <= 1e-6
    assert float((x1.grad - x2.grad).norm() / x2.grad.norm()) <= 1e-4
    # the two single-map functions with the reference's names return the same maps
    assert torch.equal(gs_loss.pixelwise_l1_with_mask(a, b, mask), l1.detach())
    assert torch.equal(gs_loss.pixelwise_ssim_with_mask(a, b, mask), ss.detach())


def test_rejects_cpu_and_mismatched_inputs():
    import gs_loss
    with pytest.raises(RuntimeError):
        gs_loss.pixelwise_l1_ssim_with_mask(torch.zeros(3, 8, 8), torch.zeros(3, 8, 8), None)
    with pytest.raises(RuntimeError):
        gs_loss.pixelwise_l1_ssim_with_mask(torch.zeros(3, 8, 8, device=DEV), torch.zeros(3, 8, 9, device=DEV), None)
