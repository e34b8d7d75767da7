"""Seeded synthetic scenes and pinhole cameras for the benchmark and the parity tests.

Camera matrices follow the reference's conventions (scene/cameras.py:59-63,
utils/graphics_utils.py:38-84): `world_view_transform` is the transposed world-to-camera
matrix, `full_proj_transform` is its fp32 product with the transposed projection
matrix (znear 0.01, zfar 100, z sign +1), `projection_matrix_inv` is the transposed
camera-to-world matrix (inverted in float64, cast to fp32) and `camera_center` is row 3
of the inverse of `world_view_transform`.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, Optional

import numpy as np
import torch


@dataclass
class Camera:
    image_width: int
    image_height: int
    FoVx: float
    FoVy: float
    world_view_transform: torch.Tensor   # (4,4) = W2C^T
    projection_matrix: torch.Tensor      # (4,4) = P^T
    full_proj_transform: torch.Tensor    # (4,4)
    projection_matrix_inv: torch.Tensor  # (4,4) = C2W^T
    camera_center: torch.Tensor          # (3,)
    uid: int = 0

    @property
    def tanfovx(self) -> float:
        return math.tan(self.FoVx * 0.5)

    @property
    def tanfovy(self) -> float:
        return math.tan(self.FoVy * 0.5)

    def to(self, device) -> "Camera":
        return Camera(self.image_width, self.image_height, self.FoVx, self.FoVy,
                      self.world_view_transform.to(device), self.projection_matrix.to(device),
                      self.full_proj_transform.to(device), self.projection_matrix_inv.to(device),
                      self.camera_center.to(device), self.uid)


def _projection(znear: float, zfar: float, fovx: float, fovy: float) -> torch.Tensor:
    tan_y, tan_x = math.tan(fovy / 2), math.tan(fovx / 2)
    top, right = tan_y * znear, tan_x * znear
    bottom, left = -top, -right
    P = torch.zeros(4, 4)
    P[0, 0] = 2.0 * znear / (right - left)
    P[1, 1] = 2.0 * znear / (top - bottom)
    P[0, 2] = (right + left) / (right - left)
    P[1, 2] = (top + bottom) / (top - bottom)
    P[3, 2] = 1.0
    P[2, 2] = zfar / (zfar - znear)
    P[2, 3] = -(zfar * znear) / (zfar - znear)
    return P


def camera_from_w2c(w2c: np.ndarray, width: int, height: int, fovx: float, fovy: Optional[float] = None) -> Camera:
    """w2c: (4,4) float64 world-to-camera matrix (x right, y down, z forward)."""
    if fovy is None:
        focal = width / (2.0 * math.tan(fovx / 2))
        fovy = 2.0 * math.atan(height / (2.0 * focal))
    wvt = torch.tensor(np.float32(w2c)).transpose(0, 1).contiguous()
    proj = _projection(0.01, 100.0, fovx, fovy).transpose(0, 1).contiguous()
    full = wvt.unsqueeze(0).bmm(proj.unsqueeze(0)).squeeze(0).contiguous()
    center = wvt.inverse()[3, :3].contiguous()
    c2w = np.linalg.inv(np.asarray(w2c, dtype=np.float64))
    pinv = torch.tensor(c2w, dtype=torch.float32).transpose(0, 1).contiguous()
    return Camera(width, height, fovx, fovy, wvt, proj, full, pinv, center)


def look_at_camera(eye, target, up, width: int, height: int, fovx_deg: float) -> Camera:
    eye, target, up = (np.asarray(v, dtype=np.float64) for v in (eye, target, up))
    fwd = target - eye
    fwd /= np.linalg.norm(fwd)
    right = np.cross(fwd, up)
    right /= np.linalg.norm(right)
    down = np.cross(fwd, right)
    R = np.stack([right, down, fwd], axis=0)  # rows: camera axes in world coordinates
    w2c = np.eye(4)
    w2c[:3, :3] = R
    w2c[:3, 3] = -R @ eye
    return camera_from_w2c(w2c, width, height, math.radians(fovx_deg))


def _attributes(n: int, gen: torch.Generator, device, scale_shift: float = 0.0,
                geometry_only: bool = False) -> Dict[str, torch.Tensor]:
    """Scales exp(N(-4, 0.5^2)) (+ scale_shift in log space), unit quaternions, opacity
    sigmoid(N(0,1)), SH degree 3: DC ~ N(0.5, 0.2^2), 45 remaining coefficients ~ N(0, 0.2^2).
    geometry_only stops after the scales (the first draw), which with the positions is all a
    partition needs."""
    kw = dict(generator=gen, device=device, dtype=torch.float32)
    scales = torch.exp(torch.randn(n, 3, **kw).mul_(0.5).add_(-4.0 + scale_shift))
    if geometry_only:
        return dict(scales=scales)
    rot = torch.randn(n, 4, **kw)
    rot = rot / rot.norm(dim=1, keepdim=True)
    opacity = torch.sigmoid(torch.randn(n, 1, **kw))
    shs = torch.randn(n, 16, 3, **kw).mul_(0.2)
    shs[:, 0, :] += 0.5
    return dict(scales=scales, rotations=rot, opacity=opacity, shs=shs)


def cube_scene(n: int, seed: int, device="cpu", geometry_only: bool = False) -> Dict[str, torch.Tensor]:
    """Config 0: positions uniform in [-1,1]^3 centred 4 units down +z."""
    gen = torch.Generator(device=device).manual_seed(seed)
    xyz = torch.rand(n, 3, generator=gen, device=device) * 2.0 - 1.0
    xyz[:, 2] += 4.0
    out = _attributes(n, gen, device, geometry_only=geometry_only)
    out["xyz"] = xyz
    return out


def garden_scene(n: int, seed: int, device="cpu", scale_shift: float = 0.0,
                 geometry_only: bool = False) -> Dict[str, torch.Tensor]:
    """Configs 1-3: 70 % on a noisy ground plane (x,y uniform over 20x20, z ~ N(0,0.05^2)),
    30 % on an upper hemisphere shell of radius 10 with N(0,0.3^2) radial jitter."""
    gen = torch.Generator(device=device).manual_seed(seed)
    n_ground = int(round(0.7 * n))
    n_shell = n - n_ground
    kw = dict(generator=gen, device=device, dtype=torch.float32)
    ground = torch.empty(n_ground, 3, device=device)
    ground[:, :2] = torch.rand(n_ground, 2, **kw) * 20.0 - 10.0
    ground[:, 2] = torch.randn(n_ground, **kw) * 0.05
    d = torch.randn(n_shell, 3, **kw)
    d = d / d.norm(dim=1, keepdim=True)
    d[:, 2] = d[:, 2].abs()
    radius = 10.0 + torch.randn(n_shell, 1, **kw) * 0.3
    shell = d * radius
    out = _attributes(n, gen, device, scale_shift, geometry_only)
    out["xyz"] = torch.cat([ground, shell], dim=0)
    return out


def city_scene(n: int, seed: int, device="cpu", blocks_per_side: int = 40,
               geometry_only: bool = False) -> Dict[str, torch.Tensor]:
    """Config 4: axis-aligned building boxes on a 2 km x 2 km grid (heights ~ U(5,120) m,
    Gaussians on the box surfaces) plus a ground plane (30 % of the Gaussians)."""
    gen = torch.Generator(device=device).manual_seed(seed)
    kw = dict(generator=gen, device=device, dtype=torch.float32)
    n_ground = int(round(0.3 * n))
    n_b = n - n_ground
    ground = torch.empty(n_ground, 3, device=device)
    ground[:, :2] = torch.rand(n_ground, 2, **kw) * 2000.0 - 1000.0
    ground[:, 2] = torch.randn(n_ground, **kw) * 0.05
    nb = blocks_per_side * blocks_per_side
    pitch = 2000.0 / blocks_per_side
    heights = torch.rand(nb, **kw) * 115.0 + 5.0
    half = pitch * 0.3
    which = torch.randint(0, nb, (n_b,), generator=gen, device=device)
    cx = (which % blocks_per_side).float() * pitch - 1000.0 + pitch / 2
    cy = (which // blocks_per_side).float() * pitch - 1000.0 + pitch / 2
    u = torch.rand(n_b, 3, **kw)
    face = torch.randint(0, 5, (n_b,), generator=gen, device=device)  # 4 walls + roof
    px = (u[:, 0] * 2 - 1) * half
    py = (u[:, 1] * 2 - 1) * half
    pz = u[:, 2] * heights[which]
    px = torch.where(face == 0, torch.full_like(px, half), torch.where(face == 1, torch.full_like(px, -half), px))
    py = torch.where(face == 2, torch.full_like(py, half), torch.where(face == 3, torch.full_like(py, -half), py))
    pz = torch.where(face == 4, heights[which], pz)
    blocks = torch.stack([cx + px, cy + py, pz], dim=1)
    del u, face, which, px, py, pz, cx, cy
    out = _attributes(n, gen, device, geometry_only=geometry_only)
    out["xyz"] = torch.cat([ground, blocks], dim=0)
    return out


# name -> (builder, number of Gaussians, resolution, bvh depth, camera, backward?)
CONFIGS = {
    "C0": dict(n=100_000, width=512, height=512, bvh_depth=0, seed=1000, backward=True),
    "C1": dict(n=5_600_000, width=1600, height=1036, bvh_depth=2, seed=1001, backward=True),
    "C2": dict(n=5_600_000, width=5185, height=3359, bvh_depth=2, seed=1001, backward=True),
    "C3": dict(n=62_900_000, width=1600, height=1036, bvh_depth=4, seed=1003, backward=True),
    "C4": dict(n=217_300_000, width=1920, height=1080, bvh_depth=5, seed=1004, backward=False),
}


def make_config(name: str, device="cpu", shrink: float = 1.0, resolution_scale: float = 1.0,
                geometry_only: bool = False):
    """Returns (scene dict, Camera, config dict).  `shrink` divides the Gaussian count and
    `resolution_scale` multiplies the image size, for tests that need a small instance of
    the same distribution.  The generator lives on `device`: a scene made on the GPU has the same
    distribution as, but other values than, the one made on the host from the same seed.
    geometry_only: positions and scales alone (the same values as in the full scene)."""
    cfg = dict(CONFIGS[name])
    cfg["name"] = name
    n = max(16, int(cfg["n"] / shrink))
    w = max(16, int(round(cfg["width"] * resolution_scale)))
    h = max(16, int(round(cfg["height"] * resolution_scale)))
    cfg.update(n=n, width=w, height=h)
    if name == "C0":
        scene = cube_scene(n, cfg["seed"], device, geometry_only=geometry_only)
        cam = look_at_camera((0, 0, 0), (0, 0, 1), (0, -1, 0), w, h, 60.0)
    elif name in ("C1", "C2"):
        scene = garden_scene(n, cfg["seed"], device, geometry_only=geometry_only)
        cam = look_at_camera((6.0, 0.0, 2.0), (0, 0, 0), (0, 0, 1), w, h, 60.0)
    elif name == "C3":
        scene = garden_scene(n, cfg["seed"], device, scale_shift=-math.log(math.sqrt(11.0)), geometry_only=geometry_only)
        cam = look_at_camera((6.0, 0.0, 2.0), (0, 0, 0), (0, 0, 1), w, h, 60.0)
    elif name == "C4":
        scene = city_scene(n, cfg["seed"], device, geometry_only=geometry_only)
        cam = look_at_camera((0.0, -300.0, 300.0), (0, 0, 0), (0, 0, 1), w, h, 60.0)
    else:
        raise KeyError(name)
    return scene, cam, cfg
