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
    return orc.settings_from_camera(cam, range_low, range_up, bg, sh_degree, scale_modifier)


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


def check_binning_against(st, geom, binning, P, R, W, H):
    """The library's binning state against the checker's, bit for bit.  The library sorts the
    Gaussians by depth first and the (Gaussian, tile) instances by tile afterwards; the checker
    follows the reference (one stable sort of instances on (tile << 32) | depth bits).  Both must
    give the same lists, and the 64-bit keys of the reference are rebuilt from the parts."""
    from retinags_amd import _capi
    g = _capi.geom_layout(P)
    touched = view_ws(geom, g["tiles_touched"], P, np.uint32)
    depth_bits = view_ws(geom, g["depths"], P, np.uint32)
    visible = np.flatnonzero(touched != 0).astype(np.uint32)
    n_vis = int(view_ws(geom, g["visible_count"], 1, np.uint32)[0])
    assert n_vis == len(visible)
    order = view_ws(geom, g["depth_order"], P, np.uint32)[:n_vis]
    assert np.array_equal(order, visible[np.argsort(depth_bits[visible], kind="stable")])
    in_order = view_ws(geom, g["point_offsets"], P, np.uint32)[:n_vis]
    assert np.array_equal(in_order, np.cumsum(touched[order].astype(np.uint64)).astype(np.uint32))
    if R == 0:
        return
    b = _capi.binning_layout(R, W, H)
    tiles = view_ws(binning, b["keys_sorted"], R, np.uint32) & np.uint32(0xFFFFFF)   # strip bits ride above the tile
    vals = view_ws(binning, b["values_sorted"], R, np.uint32)
    assert np.array_equal(vals, st.point_list)
    assert np.array_equal((tiles.astype(np.uint64) << np.uint64(32)) | depth_bits[vals].astype(np.uint64), st.keys)
