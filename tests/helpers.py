"""Shared pieces of the parity tests: the same seeded inputs as numpy arrays for the CPU
checker and as device tensors for the HIP library, and the comparison rules."""
import math
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import rgs_oracle as orc  # noqa: E402  (test infrastructure)
from retinags_amd.harness import scenes  # noqa: E402

# Tolerances of the parity contract.
IMAGE_TOL = 1e-4       # max-abs, rendered RGB / depth-weight / accumulated alpha
GRAD_TOL = 1e-3        # relative L2, every gradient tensor
# A pixel whose nearest blend decision (alpha vs 1/255, T(1-alpha) vs 1e-4) sits closer to
# its threshold than this relative distance may flip with the last bit of exp(); such pixels
# are compared separately and must stay rare.
DECISION_MARGIN = 2e-5
MAX_BORDERLINE_FRACTION = 2e-4


def np32(t):
    return np.ascontiguousarray(t.detach().cpu().numpy().astype(np.float32))


def oracle_settings(cam, range_low, range_up, bg, sh_degree=3, scale_modifier=1.0):
    return orc.Settings(
        image_height=cam.image_height, image_width=cam.image_width, tanfovx=math.tan(cam.FoVx * 0.5),
        tanfovy=math.tan(cam.FoVy * 0.5), bg=np32(bg), scale_modifier=scale_modifier,
        viewmatrix=np32(cam.world_view_transform), projmatrix=np32(cam.full_proj_transform),
        projmatrix_inv=np32(cam.projection_matrix_inv), range_low=np32(range_low), range_up=np32(range_up),
        sh_degree=sh_degree, campos=np32(cam.camera_center))


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64).ravel()
    b = np.asarray(b, dtype=np.float64).ravel()
    den = np.linalg.norm(b)
    if den == 0:
        return float(np.linalg.norm(a))
    return float(np.linalg.norm(a - b) / den)


def view_ws(buf, offset, count, dtype):
    """Typed view into a byte workspace tensor, as numpy."""
    nbytes = count * np.dtype(dtype).itemsize
    raw = buf[offset:offset + nbytes].cpu().numpy()
    return raw.view(dtype)
