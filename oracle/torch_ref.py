"""Independent torch restatement of the differentiable parts of the rasterizer.

TEST INFRASTRUCTURE ONLY.  Written from the textbook formulation (EWA
splatting with batched 3x3 matrix products, real spherical harmonics, front to
back alpha compositing), not from the op-by-op order of the C++ oracle, so the
two can disagree when either one drops a term, flips a sign or transposes an
operand.  Run it in float64: autograd through it gives the gradients the
fp32 oracle and the GPU kernels are checked against.

Conventions as CityGS-X passes them: viewmatrix V and projmatrix PM are (4,4),
row-vector form (p_view = [p,1] @ V), see scene/cameras.py:124-140.
"""
import math

import torch

C0 = 0.28209479177387814
C1 = 0.4886025119029199
C2 = [1.0925484305920792, -1.0925484305920792, 0.31539156525252005, -1.0925484305920792, 0.5462742152960396]
C3 = [-0.5900435899266435, 2.890611442640554, -0.4570457994644658, 0.3731763325901154, -0.4570457994644658,
      1.445305721320277, -0.5900435899266435]


def rotation_from_quaternion(q):
    """Textbook rotation matrix of an (r,x,y,z) quaternion, NOT normalised
    (forward.cu:128 keeps the raw quaternion)."""
    r, x, y, z = q.unbind(-1)
    R = torch.stack([
        1 - 2 * (y * y + z * z), 2 * (x * y - r * z), 2 * (x * z + r * y),
        2 * (x * y + r * z), 1 - 2 * (x * x + z * z), 2 * (y * z - r * x),
        2 * (x * z - r * y), 2 * (y * z + r * x), 1 - 2 * (x * x + y * y)], dim=-1)
    return R.reshape(q.shape[:-1] + (3, 3))


def covariance3d(scales, rotations, mod=1.0):
    R = rotation_from_quaternion(rotations)
    S = torch.diag_embed(scales * mod)
    M = R @ S
    return M @ M.transpose(-1, -2)


def sh_basis(dirs, degree):
    x, y, z = dirs.unbind(-1)
    one = torch.ones_like(x)
    b = [C0 * one]
    if degree > 0:
        b += [-C1 * y, C1 * z, -C1 * x]
    if degree > 1:
        xx, yy, zz, xy, yz, xz = x * x, y * y, z * z, x * y, y * z, x * z
        b += [C2[0] * xy, C2[1] * yz, C2[2] * (2 * zz - xx - yy), C2[3] * xz, C2[4] * (xx - yy)]
    if degree > 2:
        b += [C3[0] * y * (3 * xx - yy), C3[1] * xy * z, C3[2] * y * (4 * zz - xx - yy),
              C3[3] * z * (2 * zz - 3 * xx - 3 * yy), C3[4] * x * (4 * zz - xx - yy), C3[5] * z * (xx - yy),
              C3[6] * x * (xx - 3 * yy)]
    return torch.stack(b, dim=-1)


def sh_colour(means, campos, shs, degree):
    """shs (P,M,3) -> rgb (P,3) clamped at zero, and the clamp mask."""
    d = means - campos
    d = d / d.norm(dim=-1, keepdim=True)
    B = sh_basis(d, degree)  # (P, (deg+1)^2)
    raw = (B.unsqueeze(-1) * shs[:, : B.shape[-1], :]).sum(dim=1) + 0.5
    return torch.clamp_min(raw, 0.0), raw < 0


def preprocess(means, scales, rotations, opacities, V, PM, W, H, tanx, tany, shs=None, campos=None, degree=3, mod=1.0):
    """Geometry of forward.cu:183-258 in matrix form.  Returns a dict with
    means2D, depths, cov2D (a,b,c), conic_opacity, radius_f (before ceil->int), valid mask, rgb."""
    P = means.shape[0]
    fx = W / (2.0 * tanx)
    fy = H / (2.0 * tany)
    ones = torch.ones(P, 1, dtype=means.dtype)
    hom = torch.cat([means, ones], dim=1) @ PM
    pw = 1.0 / (hom[:, 3] + 1e-7)
    ndc = hom[:, :3] * pw[:, None]
    t = means @ V[:3, :3] + V[3, :3]
    tz = t[:, 2]
    in_front = tz > 0
    limx, limy = 1.3 * tanx, 1.3 * tany
    # Outside the +-1.3 tan(fov) guard band the clamped value is used as a constant:
    # backward.cu:101-102,187-189 zeroes the x/y mean gradient there and keeps the
    # z gradient of an unclamped formula, which is what detach() reproduces.
    ux, uy = t[:, 0] / tz, t[:, 1] / tz
    in_x = (ux >= -limx) & (ux <= limx)
    in_y = (uy >= -limy) & (uy <= limy)
    tx = torch.where(in_x, t[:, 0], (torch.clamp(ux, -limx, limx) * tz).detach())
    ty = torch.where(in_y, t[:, 1], (torch.clamp(uy, -limy, limy) * tz).detach())
    zero = torch.zeros_like(tz)
    J = torch.stack([torch.stack([fx / tz, zero, -fx * tx / (tz * tz)], -1),
                     torch.stack([zero, fy / tz, -fy * ty / (tz * tz)], -1)], dim=1)  # (P,2,3)
    Wm = V[:3, :3].transpose(0, 1)  # world -> camera rotation acting on column vectors
    Sigma = covariance3d(scales, rotations, mod)
    A = J @ Wm  # (P,2,3)
    cov = A @ Sigma @ A.transpose(-1, -2)
    a = cov[:, 0, 0] + 0.3
    b = cov[:, 0, 1]
    c = cov[:, 1, 1] + 0.3
    det = a * c - b * b
    conic = torch.stack([c / det, -b / det, a / det], dim=-1)
    mid = 0.5 * (a + c)
    lam = mid + torch.sqrt(torch.clamp_min(mid * mid - det, 0.1))
    radius_f = 3.0 * torch.sqrt(lam)
    px = ((ndc[:, 0] + 1.0) * W - 1.0) * 0.5
    py = ((ndc[:, 1] + 1.0) * H - 1.0) * 0.5
    out = dict(ndc=ndc, guard=in_x & in_y, means2D=torch.stack([px, py], -1), depths=tz, cov2D=torch.stack([a, b, c], -1),
               conic_opacity=torch.cat([conic, opacities.reshape(P, 1)], dim=1), radius_f=radius_f,
               in_front=in_front, det=det, Sigma=Sigma)
    if shs is not None:
        out["rgb"], out["clamped"] = sh_colour(means, campos, shs, degree)
    return out


def render(means2D, conic_opacity, rgb, all_map, ranges, point_list, bg, W, H, tanx, tany, render_geo=True):
    """Front-to-back compositing per 16x16 tile (forward.cu:318-436), vectorised
    over the pixels of a tile.  ranges/point_list come from the binning stage
    and are treated as constants.  Returns color (3,H,W), all_map (5,H,W),
    plane_depth (1,H,W), final_T (H,W), n_contrib (H,W)."""
    dt = means2D.dtype
    fx = W / (2.0 * tanx)
    fy = H / (2.0 * tany)
    gx, gy = (W + 15) // 16, (H + 15) // 16
    color = torch.zeros(3, H, W, dtype=dt)
    omap = torch.zeros(5, H, W, dtype=dt)
    depth = torch.zeros(1, H, W, dtype=dt)
    final_T = torch.ones(H, W, dtype=dt)
    n_contrib = torch.zeros(H, W, dtype=torch.int64)
    bg = bg.to(dt)
    for tyi in range(gy):
        for txi in range(gx):
            tile = tyi * gx + txi
            r0, r1 = int(ranges[tile][0]), int(ranges[tile][1])
            y0, y1 = tyi * 16, min(H, tyi * 16 + 16)
            x0, x1 = txi * 16, min(W, txi * 16 + 16)
            ys, xs = torch.meshgrid(torch.arange(y0, y1, dtype=dt), torch.arange(x0, x1, dtype=dt), indexing="ij")
            pxy = torch.stack([xs.reshape(-1), ys.reshape(-1)], -1)  # (npx,2)
            npx = pxy.shape[0]
            if r1 > r0:
                ids = torch.as_tensor(point_list[r0:r1].astype("int64"))
                d = means2D[ids][None, :, :] - pxy[:, None, :]  # (npx,n,2)
                co = conic_opacity[ids]
                power = -0.5 * (co[None, :, 0] * d[..., 0] ** 2 + co[None, :, 2] * d[..., 1] ** 2) \
                    - co[None, :, 1] * d[..., 0] * d[..., 1]
                alpha = torch.clamp_max(co[None, :, 3] * torch.exp(power), 0.99)
                keep = (power <= 0) & (alpha >= 1.0 / 255.0)
                alpha = torch.where(keep, alpha, torch.zeros_like(alpha))
                T_incl = torch.cumprod(1 - alpha, dim=1)
                T_excl = torch.cat([torch.ones(npx, 1, dtype=dt), T_incl[:, :-1]], dim=1)
                # the first kept Gaussian that would push T below 1e-4 stops the pixel (and is not blended)
                stop = keep & (T_incl < 1e-4)
                alive = torch.cumsum(stop.to(torch.int64), dim=1) == 0
                use = keep & alive
                w = torch.where(use, alpha * T_excl, torch.zeros_like(alpha))
                Tf = torch.prod(torch.where(use, 1 - alpha, torch.ones_like(alpha)), dim=1)
                col = w @ rgb[ids]
                mp = w @ all_map[ids]
                idx = torch.arange(1, r1 - r0 + 1)[None, :].expand(npx, -1)
                last = torch.where(use, idx, torch.zeros_like(idx)).max(dim=1).values
            else:
                Tf = torch.ones(npx, dtype=dt)
                col = torch.zeros(npx, 3, dtype=dt)
                mp = torch.zeros(npx, 5, dtype=dt)
                last = torch.zeros(npx, dtype=torch.int64)
            hh, ww = y1 - y0, x1 - x0
            color[:, y0:y1, x0:x1] = (col + Tf[:, None] * bg[None, :]).t().reshape(3, hh, ww)
            final_T[y0:y1, x0:x1] = Tf.reshape(hh, ww)
            n_contrib[y0:y1, x0:x1] = last.reshape(hh, ww)
            if render_geo:
                omap[:, y0:y1, x0:x1] = mp.t().reshape(5, hh, ww)
                rayx = (pxy[:, 0] - W * 0.5) / fx
                rayy = (pxy[:, 1] - H * 0.5) / fy
                den = -(mp[:, 0] * rayx + mp[:, 1] * rayy + mp[:, 2] + 1e-8)
                depth[0, y0:y1, x0:x1] = (mp[:, 4] / den).reshape(hh, ww)
    return dict(color=color, out_all_map=omap, out_plane_depth=depth, final_T=final_T, n_contrib=n_contrib)
