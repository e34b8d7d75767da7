"""Independent float64 mathematics used to pin the CPU checker (oracle/).

Nothing here is derived from the checker's source: projection is a plain matrix product,
the covariance is R diag(s^2) R^T pushed through the EWA Jacobian, spherical harmonics come
from scipy's complex harmonics, tile coverage is brute force, and the renderer is a
differentiable torch program whose gradients come from autograd.  Where the reference
deliberately deviates from the true gradient, the deviation is modelled here as what it is: the
0.99 clamp as a straight-through estimator, the guard-frustum clamp as a constant to the backward
pass (detached), the quaternion used as given; only the 1e-7 in the determinant's reciprocal is
left out (scenes with determinants far above it).
"""
import math

import numpy as np
import torch


def quat_to_rotmat(q):
    """Standard rotation matrix of a quaternion (r, x, y, z), used without normalising."""
    r, x, y, z = q[..., 0], q[..., 1], q[..., 2], q[..., 3]
    rows = [
        torch.stack([1 - 2 * (y * y + z * z), 2 * (x * y - r * z), 2 * (x * z + r * y)], -1),
        torch.stack([2 * (x * y + r * z), 1 - 2 * (x * x + z * z), 2 * (y * z - r * x)], -1),
        torch.stack([2 * (x * z - r * y), 2 * (y * z + r * x), 1 - 2 * (x * x + y * y)], -1),
    ]
    return torch.stack(rows, -2)


def covariance3d(scales, quats, mod=1.0):
    R = quat_to_rotmat(quats)
    S2 = torch.diag_embed((mod * scales) ** 2)
    return R @ S2 @ R.transpose(-1, -2)


def real_sh_basis(dirs, degree=3):
    """(n, (degree+1)^2) real spherical harmonics in the sign convention of 3D Gaussian
    splatting: index l*l + l + m, equal to (-1)^m times the usual real harmonics."""
    try:  # scipy >= 1.15: sph_harm_y(l, m, polar, azimuth)
        from scipy.special import sph_harm_y
        sph_harm = lambda m, l, azimuth, polar: sph_harm_y(l, m, polar, azimuth)
    except ImportError:
        from scipy.special import sph_harm
    d = np.asarray(dirs, dtype=np.float64)
    d = d / np.linalg.norm(d, axis=1, keepdims=True)
    theta = np.arctan2(d[:, 1], d[:, 0])          # azimuth
    phi = np.arccos(np.clip(d[:, 2], -1.0, 1.0))  # polar angle
    out = np.zeros((d.shape[0], (degree + 1) ** 2))
    for l in range(degree + 1):
        for m in range(-l, l + 1):
            Y = sph_harm(abs(m), l, theta, phi)
            if m < 0:
                v = math.sqrt(2.0) * (-1) ** m * Y.imag
            elif m > 0:
                v = math.sqrt(2.0) * (-1) ** m * Y.real
            else:
                v = Y.real
            out[:, l * l + l + m] = (-1) ** m * v
    return out


def project(means, view_t, proj_t):
    """view_t / proj_t are the transposed matrices the rasterizer receives (row-vector
    convention): p_view = [x y z 1] @ view_t."""
    hom = torch.cat([means, torch.ones_like(means[:, :1])], dim=1)
    p_view = hom @ view_t
    p_clip = hom @ proj_t
    return p_view, p_clip


def ewa_cov2d(means, cov3d, view_t, W, H, tanx, tany):
    """J W Sigma W^T J^T + 0.3 I with the 1.3 x guard-frustum clamp of the view-space mean."""
    hom = torch.cat([means, torch.ones_like(means[:, :1])], dim=1)
    t = (hom @ view_t)[:, :3]
    fx, fy = W / (2 * tanx), H / (2 * tany)
    lx, ly = 1.3 * tanx, 1.3 * tany
    tz = t[:, 2]
    # Outside the guard band the clamped coordinate is a constant to the backward pass: no gradient
    # to t.x (t.y), and none to t.z through it (K/cuda_rasterizer_hgs/backward.cu:168-176, 262-264).
    rx, ry = t[:, 0] / tz, t[:, 1] / tz
    cx, cy = torch.clamp(rx, -lx, lx), torch.clamp(ry, -ly, ly)
    tx = torch.where(cx == rx, t[:, 0], (cx * tz).detach())
    ty = torch.where(cy == ry, t[:, 1], (cy * tz).detach())
    zero = torch.zeros_like(tz)
    J = torch.stack([torch.stack([fx / tz, zero, -fx * tx / tz ** 2], -1),
                     torch.stack([zero, fy / tz, -fy * ty / tz ** 2], -1)], -2)   # (n,2,3)
    Wm = view_t[:3, :3].transpose(0, 1)                                           # world -> view rotation
    A = J @ Wm
    cov = A @ cov3d @ A.transpose(-1, -2)
    return cov + 0.3 * torch.eye(2, dtype=cov.dtype)


def tile_rect_bruteforce(px, py, radius, W, H):
    """Tiles [x0,x1) x [y0,y1) of a 16-pixel grid touched by the square of half-size `radius`
    around (px, py), by the rule tile index = floor(coordinate / 16) clamped to the grid
    (upper edge: first tile index whose start is beyond px + radius)."""
    gx, gy = (W + 15) // 16, (H + 15) // 16
    x0 = min(gx, max(0, int(math.floor((px - radius) / 16.0)) if px - radius >= 0 else 0))
    y0 = min(gy, max(0, int(math.floor((py - radius) / 16.0)) if py - radius >= 0 else 0))
    ux, uy = (px + radius + 15.0) / 16.0, (py + radius + 15.0) / 16.0
    x1 = min(gx, max(0, int(math.floor(ux)) if ux >= 0 else 0))
    y1 = min(gy, max(0, int(math.floor(uy)) if uy >= 0 else 0))
    return x0, y0, x1, y1


def render_reference(params, cam, W, H, low, up, bg, sh_degree=3, mod=1.0):
    """Differentiable float64 half-Gaussian renderer, one pixel at a time.

    params: dict of float64 torch tensors (xyz, scales, rotations, opacity (n,1), shs (n,16,3)).
    cam: dict with view_t, proj_t, c2w_t (4,4 float64, transposed convention), campos (3,),
    tanx, tany.  Returns colour (3,H,W), depth (1,H,W), alpha (1,H,W) and, for tests of the
    integer stages, per-Gaussian (radius, rect, visible).
    """
    xyz, scales, quats, opac, shs = (params[k] for k in ("xyz", "scales", "rotations", "opacity", "shs"))
    n = xyz.shape[0]
    view_t, proj_t, c2w_t = cam["view_t"], cam["proj_t"], cam["c2w_t"]
    tanx, tany = cam["tanx"], cam["tany"]
    p_view, p_clip = project(xyz, view_t, proj_t)
    depth = p_view[:, 2]
    w_clip = p_clip[:, 3]
    ndc = p_clip[:, :2] / (w_clip[:, None] + 1e-7)
    pix = torch.stack([((ndc[:, 0] + 1) * W - 1) * 0.5, ((ndc[:, 1] + 1) * H - 1) * 0.5], -1)
    if pix.requires_grad:
        pix.retain_grad()   # the blend is the only differentiable reader of the pixel centres: see aux["pix_node"]
    cov3d = covariance3d(scales, quats, mod)
    cov2d = ewa_cov2d(xyz, cov3d, view_t, W, H, tanx, tany)
    conic = torch.linalg.inv(cov2d)
    with torch.no_grad():
        # extent: 3 sigma of the larger eigenvalue, where the half-gap between the two
        # eigenvalues is floored at sqrt(0.1) (the forward's definition of the radius)
        lam = torch.linalg.eigvalsh(cov2d)
        mid = 0.5 * (lam[:, 0] + lam[:, 1])
        half_gap = 0.5 * (lam[:, 1] - lam[:, 0])
        radius = torch.ceil(3 * torch.sqrt(mid + torch.sqrt(torch.clamp(half_gap ** 2, min=0.1))))
        visible = depth > 0.2
        rects = []
        for i in range(n):
            rc = tile_rect_bruteforce(float(pix[i, 0]), float(pix[i, 1]), float(radius[i]), W, H)
            rects.append(rc)
            if (rc[2] - rc[0]) * (rc[3] - rc[1]) == 0:
                visible[i] = False
    # colour
    dirs = xyz - cam["campos"][None]
    dirs = dirs / dirs.norm(dim=1, keepdim=True)
    basis = torch.from_numpy(real_sh_basis(dirs.detach().numpy(), 3))
    # the basis is a polynomial in the unit direction; rebuild it differentiably from scipy's
    # values by evaluating the same polynomials symbolically is not possible, so the
    # view-direction gradient is carried by an explicit polynomial form checked against scipy
    basis_t = sh_polynomials(dirs)
    assert torch.allclose(basis_t.detach(), basis, atol=1e-12)
    ncoef = (sh_degree + 1) ** 2
    rgb = torch.einsum("nk,nkc->nc", basis_t[:, :ncoef], shs[:, :ncoef, :]) + 0.5
    rgb = torch.clamp(rgb, min=0.0)

    order = torch.argsort(depth.detach(), stable=True)
    order = [int(i) for i in order if bool(visible[i])]
    gx = (W + 15) // 16
    color = torch.zeros(3, H, W, dtype=torch.float64)
    out_depth = torch.zeros(1, H, W, dtype=torch.float64)
    out_alpha = torch.zeros(1, H, W, dtype=torch.float64)
    lists = {}
    for py in range(H):
        for px in range(W):
            tx, ty = px // 16, py // 16
            key = (tx, ty)
            if key not in lists:
                lists[key] = [i for i in order if rects[i][0] <= tx < rects[i][2] and rects[i][1] <= ty < rects[i][3]]
            ids = lists[key]
            if not ids:
                color[:, py, px] = bg
                continue
            idt = torch.tensor(ids)
            d = pix[idt] - torch.tensor([float(px), float(py)], dtype=torch.float64)
            cn = conic[idt]
            power = -0.5 * (cn[:, 0, 0] * d[:, 0] ** 2 + cn[:, 1, 1] * d[:, 1] ** 2) - cn[:, 0, 1] * d[:, 0] * d[:, 1]
            G = torch.exp(power)
            # 0.99 clamp with a straight-through gradient
            raw = opac[idt, 0] * G
            alpha = raw + (torch.clamp(raw, max=0.99) - raw).detach()
            # ray point at each Gaussian's clip-w, in world space
            ndcx = (2.0 * px + 1.0) / W - 1.0
            ndcy = (2.0 * py + 1.0) / H - 1.0
            wv = w_clip[idt].detach()
            ph = torch.stack([ndcx * (wv + 1e-7) * tanx, ndcy * (wv + 1e-7) * tany, wv, torch.ones_like(wv)], -1)
            pw = ph @ c2w_t
            inbox = ((pw[:, :3] > low[None]) & (pw[:, :3] <= up[None])).all(dim=1)
            with torch.no_grad():
                use = (power <= 0) & (alpha >= 1.0 / 255.0) & inbox
                keep = torch.zeros_like(use)
                T = 1.0
                for j in range(len(ids)):
                    if not bool(use[j]):
                        continue
                    tt = T * (1 - float(alpha[j]))
                    if tt < 1e-4:
                        break
                    keep[j] = True
                    T = tt
            a = alpha * keep
            Tbefore = torch.cumprod(torch.cat([torch.ones(1, dtype=torch.float64), 1 - a[:-1]]), 0)
            wgt = a * Tbefore
            Tend = Tbefore[-1] * (1 - a[-1])
            color[:, py, px] = (wgt[:, None] * rgb[idt]).sum(0) + Tend * bg
            out_depth[0, py, px] = (wgt * depth[idt]).sum()
            out_alpha[0, py, px] = wgt.sum()
    aux = dict(radius=radius, rects=rects, visible=visible, pix=pix.detach(), pix_node=pix, conic=conic.detach(),
               depth=depth.detach(), rgb=rgb.detach(), cov3d=cov3d.detach(), cov2d=cov2d.detach())
    return color, out_depth, out_alpha, aux


def sh_polynomials(d):
    """The 16 real harmonics (3DGS sign convention) as polynomials of a unit vector, written
    from the standard closed forms N_lm * P_lm and checked against scipy by the caller."""
    x, y, z = d[:, 0], d[:, 1], d[:, 2]
    pi = math.pi
    c0 = 0.5 * math.sqrt(1 / pi)
    c1 = math.sqrt(3 / (4 * pi))
    c2a = 0.5 * math.sqrt(15 / pi)
    c2b = 0.25 * math.sqrt(5 / pi)
    c2c = 0.25 * math.sqrt(15 / pi)
    c3a = 0.25 * math.sqrt(35 / (2 * pi))
    c3b = 0.5 * math.sqrt(105 / pi)
    c3c = 0.25 * math.sqrt(21 / (2 * pi))
    c3d = 0.25 * math.sqrt(7 / pi)
    c3e = 0.25 * math.sqrt(105 / pi)
    cols = [
        c0 * torch.ones_like(x),
        -c1 * y, c1 * z, -c1 * x,
        c2a * x * y, -c2a * y * z, c2b * (3 * z * z - 1), -c2a * x * z, c2c * (x * x - y * y),
        -c3a * y * (3 * x * x - y * y), c3b * x * y * z, -c3c * y * (5 * z * z - 1),
        c3d * z * (5 * z * z - 3), -c3c * x * (5 * z * z - 1), c3e * z * (x * x - y * y),
        -c3a * x * (x * x - 3 * y * y),
    ]
    return torch.stack(cols, -1)
