"""Writes tests/golden/half_gaussian_small.npz: seeded inputs and the CPU checker's outputs for
them (every forward stage and every gradient).  The reference holds no fixtures for this
path, so the vectors come from this repository's own checker, which tests/test_oracle_pins.py
pins against independent mathematics.  Run: python tests/golden/make_golden.py"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from helpers import np32, oracle_settings, orc, scenes  # noqa: E402


def build_case(seed, n, W, H, up):
    g = torch.Generator().manual_seed(seed)
    xyz = (torch.rand(n, 3, generator=g) * 2 - 1) * 1.2
    xyz[:, 2] = xyz[:, 2] * 0.6 + 4.0
    xyz[: n // 10, 2] -= 6.0  # some behind the camera
    scales = torch.exp(torch.randn(n, 3, generator=g) * 0.4 - 2.6)
    rot = torch.randn(n, 4, generator=g)
    rot = rot / rot.norm(dim=1, keepdim=True)
    opacity = torch.sigmoid(torch.randn(n, 1, generator=g))
    shs = torch.randn(n, 16, 3, generator=g) * 0.2
    shs[:, 0] += 0.5
    cam = scenes.look_at_camera((0.2, -0.1, 0.0), (0.0, 0.0, 4.0), (0, -1, 0), W, H, 60.0)
    low = torch.tensor([-40.0, -40.0, -40.0])
    bg = torch.tensor([0.15, 0.3, 0.45])
    s = oracle_settings(cam, low, up, bg)
    st = orc.forward(s, np32(xyz), np32(opacity), shs=np32(shs), scales=np32(scales), rotations=np32(rot),
                     want_margin=True)
    g_color = np32(torch.randn(3, H, W, generator=g) * 1e-2)
    g_depth = np32(torch.randn(1, H, W, generator=g) * 1e-2)
    g_alpha = np32(torch.randn(1, H, W, generator=g) * 1e-2)
    gr = orc.backward(s, st, g_color, g_depth, g_alpha)
    out = dict(
        xyz=np32(xyz), scales=np32(scales), rotations=np32(rot), opacity=np32(opacity), shs=np32(shs),
        viewmatrix=s.viewmatrix, projmatrix=s.projmatrix, projmatrix_inv=s.projmatrix_inv, campos=s.campos,
        range_low=s.range_low, range_up=s.range_up, bg=s.bg, tanfov=np.array([s.tanfovx, s.tanfovy], np.float64),
        size=np.array([W, H], np.int32),
        radii=st.radii, tiles_touched=st.tiles_touched, xy=st.xy, depths=st.depths, keys=st.keys,
        point_list=st.point_list, ranges=st.ranges, color=st.color, depth=st.depth, alpha=st.alpha,
        n_contrib=st.n_contrib, margin=st.margin, g_color=g_color, g_depth=g_depth, g_alpha=g_alpha)
    for k, v in gr.items():
        out["grad_" + k] = v
    return out


def main():
    cases = {"open": build_case(11, 200, 64, 56, torch.tensor([40.0, 40.0, 40.0])),
             "clipped": build_case(12, 200, 60, 50, torch.tensor([0.1, 40.0, 4.3]))}
    flat = {f"{c}/{k}": v for c, d in cases.items() for k, v in d.items()}
    path = os.path.join(HERE, "half_gaussian_small.npz")
    np.savez_compressed(path, **flat)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
