"""Seeded synthetic scenes and cameras for the rasterizer tests, smoke check and benchmark (not part of the product
package).

Cameras are built the way CityGS-X builds them (row-vector convention):
world_view_transform = W2C^T, full_proj = world_view_transform @ P^T
(utils/graphics_utils.py:42-76, scene/cameras.py:118-140), so the matrices can
be handed to GaussianRasterizationSettings unchanged.  The per-Gaussian
all_map follows gaussian_renderer/__init__.py:1501-1518.

Random draws come from one torch.Generator in a fixed order (means, log-scales,
quaternions, opacity logits, SH DC, SH rest, upstream gradients), so every
machine regenerates identical tensors from the seed.
"""
import math
from typing import NamedTuple

import numpy as np
import torch


class Camera(NamedTuple):
    image_width: int
    image_height: int
    FoVx: float
    FoVy: float
    world_view_transform: torch.Tensor  # (4,4) = W2C^T
    full_proj_transform: torch.Tensor  # (4,4)
    camera_center: torch.Tensor  # (3,)

    @property
    def tanfovx(self):
        return math.tan(self.FoVx * 0.5)

    @property
    def tanfovy(self):
        return math.tan(self.FoVy * 0.5)


def projection_matrix(znear, zfar, fovX, fovY):
    """utils/graphics_utils.py:56-76."""
    tanHalfFovY = math.tan(fovY / 2)
    tanHalfFovX = math.tan(fovX / 2)
    top = tanHalfFovY * znear
    bottom = -top
    right = tanHalfFovX * znear
    left = -right
    P = torch.zeros(4, 4)
    P[0, 0] = 2.0 * znear / (right - left)
    P[1, 1] = 2.0 * znear / (top - bottom)
    P[0, 2] = (right + left) / (right - left)
    P[1, 2] = (top + bottom) / (top - bottom)
    P[3, 2] = 1.0
    P[2, 2] = zfar / (zfar - znear)
    P[2, 3] = -(zfar * znear) / (zfar - znear)
    return P


def look_at_camera(eye, target, W, H, fovx_deg, up=(0.0, 0.0, 1.0)):
    """Pinhole camera at `eye` looking at `target` (camera +z forward, +y down)."""
    eye = np.asarray(eye, np.float64)
    f = np.asarray(target, np.float64) - eye
    f /= np.linalg.norm(f)
    upv = np.asarray(up, np.float64)
    if abs(np.dot(f, upv)) > 0.999:
        upv = np.array([0.0, 1.0, 0.0])
    x = np.cross(f, upv)
    x /= np.linalg.norm(x)
    y = np.cross(f, x)
    R = np.stack([x, y, f], axis=1)  # camera-to-world rotation, columns = camera axes
    T = -R.T @ eye
    # getWorld2View2 (utils/graphics_utils.py:42-53) with zero translate and unit scale
    Rt = np.zeros((4, 4))
    Rt[:3, :3] = R.T
    Rt[:3, 3] = T
    Rt[3, 3] = 1.0
    wvt = torch.tensor(np.float32(Rt)).transpose(0, 1).contiguous()
    fovx = math.radians(fovx_deg)
    focal = W / (2.0 * math.tan(fovx / 2))
    fovy = 2.0 * math.atan(H / (2.0 * focal))
    proj = projection_matrix(0.01, 100.0, fovx, fovy).transpose(0, 1)
    full = (wvt.unsqueeze(0).bmm(proj.unsqueeze(0))).squeeze(0).contiguous()
    center = wvt.inverse()[3, :3].contiguous()
    return Camera(W, H, fovx, fovy, wvt, full, center)


def _gaussians(gen, means, log_scale_mu, log_scale_sigma, opacity_sigma):
    P = means.shape[0]
    scales = torch.exp(torch.randn(P, 3, generator=gen) * log_scale_sigma + log_scale_mu)
    q = torch.randn(P, 4, generator=gen)
    q = q / q.norm(dim=1, keepdim=True)
    opac = torch.sigmoid(torch.randn(P, 1, generator=gen) * opacity_sigma)
    sh = torch.empty(P, 16, 3)
    sh[:, 0, :] = torch.randn(P, 3, generator=gen) * 0.3
    sh[:, 1:, :] = torch.randn(P, 15, 3, generator=gen) * 0.05
    return dict(means3D=means.contiguous(), scales=scales.contiguous(), rotations=q.contiguous(),
                opacities=opac.contiguous(), shs=sh.contiguous())


def make_scene(config, seed=0, P=None, n_views=None):
    """Returns (gaussians dict, [Camera, ...]) for BASELINE config 0..4.

    P and n_views override the config's counts (tests use reduced P with the
    same distributions).
    """
    gen = torch.Generator().manual_seed(seed)
    if config == 0:
        P = P or 50_000
        means = (torch.rand(P, 3, generator=gen) * 2 - 1) * 10.0
        g = _gaussians(gen, means, -4.0, 0.5, 1.0)
        cams = [look_at_camera((0.0, 0.0, -30.0), (0, 0, 0), 640, 480, 60.0, up=(0.0, -1.0, 0.0))]
    elif config == 1:
        P = P or 1_000_000
        u = torch.rand(P, 3, generator=gen)
        means = torch.stack([(u[:, 0] - 0.5) * 200.0, (u[:, 1] - 0.5) * 200.0, u[:, 2] * 30.0], dim=1)
        g = _gaussians(gen, means, -2.5, 0.7, 1.5)
        cams = [look_at_camera((0.0, -120.0, 120.0), (0.0, 0.0, 0.0), 1152, 864, 70.0)]
    elif config == 2:
        P = P or 4_000_000
        n_views = n_views or 4
        u = torch.rand(P, 3, generator=gen)
        zn = torch.randn(P, generator=gen) * 3.0 + 2.0
        near = torch.rand(P, generator=gen) < 0.7
        z = torch.where(near, zn, u[:, 2] * 60.0)
        means = torch.stack([(u[:, 0] - 0.5) * 1000.0, (u[:, 1] - 0.5) * 1000.0, z], dim=1)
        g = _gaussians(gen, means, -2.0, 0.8, 1.5)
        cams = []
        for v in range(n_views):
            ang = 2 * math.pi * v / n_views
            alt = 150.0 + 50.0 * v / max(1, n_views - 1)
            cams.append(look_at_camera((300.0 * math.cos(ang), 300.0 * math.sin(ang), alt), (0.0, 0.0, 0.0), 1152, 864, 70.0))
    elif config in (3, 4):
        P = P or (10_000_000 if config == 3 else 20_000_000)
        n_views = n_views or (8 if config == 3 else 4)
        u = torch.rand(P, 3, generator=gen)
        # density doubled within 10 m of the ground: mixture of a [0,10] and a [0,80] slab
        low = torch.rand(P, generator=gen) < (1.0 / 9.0)
        z = torch.where(low, u[:, 2] * 10.0, u[:, 2] * 80.0)
        means = torch.stack([(u[:, 0] - 0.5) * 2000.0, (u[:, 1] - 0.5) * 2000.0, z], dim=1)
        g = _gaussians(gen, means, -2.0, 0.8, 1.5)
        cams = []
        for v in range(n_views):
            if config == 3:
                yaw = float(torch.rand(1, generator=gen)) * 2 * math.pi
                pos = ((float(torch.rand(1, generator=gen)) - 0.5) * 1000.0, (float(torch.rand(1, generator=gen)) - 0.5) * 1000.0, 2.0)
                tgt = (pos[0] + math.cos(yaw), pos[1] + math.sin(yaw), 2.0)
                cams.append(look_at_camera(pos, tgt, 1920, 1080, 90.0))
            else:
                ang = 2 * math.pi * v / n_views
                cams.append(look_at_camera((600.0 * math.cos(ang), 600.0 * math.sin(ang), 200.0), (0.0, 0.0, 0.0), 1152, 864, 70.0))
    else:
        raise ValueError(f"unknown config {config}")
    g["seed"] = seed
    return g, cams


def upstream_grads(cam, seed=0):
    """N(0,1) upstream gradients for colour, all_map and plane depth."""
    gen = torch.Generator().manual_seed(seed + 1000)
    H, W = cam.image_height, cam.image_width
    return dict(color=torch.randn(3, H, W, generator=gen), all_map=torch.randn(5, H, W, generator=gen),
                plane_depth=torch.randn(1, H, W, generator=gen))


def quaternion_to_matrix(q):
    """Rotation matrices from (r,x,y,z) quaternions (pytorch3d.transforms convention)."""
    r, i, j, k = torch.unbind(q, -1)
    two_s = 2.0 / (q * q).sum(-1)
    o = torch.stack(
        (1 - two_s * (j * j + k * k), two_s * (i * j - k * r), two_s * (i * k + j * r),
         two_s * (i * j + k * r), 1 - two_s * (i * i + k * k), two_s * (j * k - i * r),
         two_s * (i * k - j * r), two_s * (j * k + i * r), 1 - two_s * (i * i + j * j)), -1)
    return o.reshape(q.shape[:-1] + (3, 3))


def build_all_map(means3D, scales, rotations, cam):
    """Per-Gaussian [normal_cam(3), 1, |n . p_cam|] (gaussian_renderer/__init__.py:1501-1518)."""
    wvt = cam.world_view_transform.to(means3D.device)
    center = cam.camera_center.to(means3D.device)
    Rm = quaternion_to_matrix(torch.nn.functional.normalize(rotations, p=2, dim=-1))
    idx = scales.min(dim=-1)[1][..., None, None].expand(-1, 3, -1)
    normal = Rm.gather(2, idx).squeeze(dim=2)
    to_cam = center - means3D
    neg = (normal * to_cam).sum(-1) < 0.0
    normal = torch.where(neg[:, None], -normal, normal)
    local_normal = normal @ wvt[:3, :3]
    pts_cam = means3D @ wvt[:3, :3] + wvt[3, :3]
    dist = (local_normal * pts_cam).sum(-1).abs()
    out = torch.zeros(means3D.shape[0], 5, dtype=means3D.dtype, device=means3D.device)
    out[:, :3] = local_normal
    out[:, 3] = 1.0
    out[:, 4] = dist
    return out


def make_anchor_scene(N, k=10, seed=0, feat_dim=32, input_flags=0):
    """Seeded anchors for the neural-Gaussian generation step: anchor positions, features, offsets,
    activated scalings (N,6), a camera centre and the three MLPs as nn.Linear-shaped tensors
    (scene/gaussian_model.py:131-149: Linear(feat_dim+3, feat_dim), ReLU, Linear(feat_dim, out)) drawn with
    nn.Linear's default range.  input_flags widens the first layers by the optional inputs (add_opacity_dist = 1,
    add_color_dist = 2, add_cov_dist = 4: the distance; add_level = 8: the level, :118-121).  Returns a dict; "mlps"
    is [(W1, b1, W2, b2)] in the order opacity, color, cov; "level" is the anchors' level (N, 1)."""
    gen = torch.Generator().manual_seed(1000 + seed)
    r = lambda *s: torch.rand(*s, generator=gen)
    n = lambda *s: torch.randn(*s, generator=gen)
    anchor = (r(N, 3) - 0.5) * torch.tensor([400.0, 400.0, 40.0])
    feat = n(N, feat_dim) * 0.7
    offsets = n(N, k, 3) * 0.5
    scaling = torch.exp(n(N, 6) * 0.4 - 1.0)
    campos = torch.tensor([10.0, -20.0, 120.0])
    mlps = []
    for m, out in enumerate((k, 3 * k, 7 * k)):
        width = feat_dim + 3 + ((input_flags >> m) & 1) + ((input_flags >> 3) & 1)
        a1, a2 = 1.0 / math.sqrt(width), 1.0 / math.sqrt(feat_dim)
        mlps.append(((r(feat_dim, width) * 2 - 1) * a1, (r(feat_dim) * 2 - 1) * a1,
                     (r(out, feat_dim) * 2 - 1) * a2, (r(out) * 2 - 1) * a2))
    level = torch.randint(0, 6, (N, 1), generator=gen).float()
    return {"anchor": anchor, "feat": feat, "offsets": offsets, "scaling": scaling, "campos": campos, "mlps": mlps,
            "level": level}


def neural_gaussians_torch(anchor, feat, offsets, scaling, campos, mlps, prog=None, level=None, input_flags=0):
    """generate_neural_gaussians (gaussian_renderer/__init__.py:789-899) in its default configuration, with
    torch operations in the dtype of its inputs: the comparison the fused operator is measured against.  prog
    (N, 1), if given, is the factor dist2level 'progressive' puts on the opacity (:844-848); level (N, 1) and
    input_flags (add_opacity_dist = 1, add_color_dist = 2, add_cov_dist = 4, add_level = 8) are the MLPs' optional
    inputs (:824-877)."""
    k = offsets.shape[1]
    ob_view = anchor - campos
    ob_dist = ob_view.norm(dim=1, keepdim=True)
    ob_view = ob_view / ob_dist
    lv = [level.reshape(-1, 1).to(feat.dtype)] if input_flags & 8 else []
    with_dist = torch.cat([feat, ob_view, ob_dist] + lv, dim=1)
    without = torch.cat([feat, ob_view] + lv, dim=1)

    def run(i):
        m, x = mlps[i], with_dist if (input_flags >> i) & 1 else without
        return torch.relu(x @ m[0].t() + m[1]) @ m[2].t() + m[3]

    neural_opacity = torch.tanh(run(0))
    if prog is not None:
        neural_opacity = neural_opacity * prog
    neural_opacity = neural_opacity.reshape(-1, 1)
    mask = (neural_opacity > 0.0).view(-1)
    opacity = neural_opacity[mask]
    color = torch.sigmoid(run(1)).reshape(-1, 3)
    scale_rot = run(2).reshape(-1, 7)
    cat = torch.cat([scaling, anchor], dim=-1).repeat_interleave(k, dim=0)
    masked = torch.cat([cat, color, scale_rot, offsets.reshape(-1, 3)], dim=-1)[mask]
    scaling_repeat, repeat_anchor, color, scale_rot, offs = masked.split([6, 3, 3, 7, 3], dim=-1)
    scal = scaling_repeat[:, 3:] * torch.sigmoid(scale_rot[:, :3])
    rot = torch.nn.functional.normalize(scale_rot[:, 3:7])
    xyz = repeat_anchor + offs * scaling_repeat[:, :3]
    return xyz, color, opacity, scal, rot, neural_opacity, mask
