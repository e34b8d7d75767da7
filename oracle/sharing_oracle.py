"""CPU restatement of the two scheduler routines that sit either side of the rasterizer:
which submodels a camera sees (box against view frustum, compositing order) and which
Gaussians a submodel lends to its neighbours (boundary straddlers) with the merge of the
lent rows behind a submodel's own.

TEST INFRASTRUCTURE ONLY.  Tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the shipped package must not.  Paths are relative to the
reference's root.

Pinned by tests/test_scheduling_cpu.py: the hull test by linear-programming feasibility of a
common point of the two vertex sets' convex hulls and by closed cases; the order by the pairwise
constraint every split plane imposes (of two leaves that part ways at a node, the one on the
camera's side comes first); the straddler selection by a per-Gaussian scalar loop; the merge by
its adjoint identity.
"""
from __future__ import annotations

import math
from typing import Dict, List, Sequence, Tuple

import numpy as np


# ---------------------------------------------------------------------------------------------
# box against frustum: parallel_utils/grid_utils/utils.py:14-137
# ---------------------------------------------------------------------------------------------
def space_box_vertices(range_low, range_up) -> np.ndarray:
    """The 8 vertices in the reference's order (grid_utils/utils.py:36-44)."""
    x0, y0, z0 = range_low
    x1, y1, z1 = range_up
    return np.array([(x0, y0, z0), (x0, y0, z1), (x0, y1, z1), (x0, y1, z0),
                     (x1, y0, z0), (x1, y0, z1), (x1, y1, z1), (x1, y1, z0)], dtype=np.float32)


def frustum_vertices(fovx: float, fovy: float, z_near=None, z_far=None) -> np.ndarray:
    """grid_utils/utils.py:84-112."""
    tan_y = math.tan(fovy / 2)
    tan_x = math.tan(fovx / 2)
    near = max(0.01, 0.01 if z_near is None else z_near)
    far = min(1e6, 1e6 if z_far is None else z_far)
    unit = np.array([(tan_x, tan_y, 1), (tan_x, -tan_y, 1), (-tan_x, tan_y, 1), (-tan_x, -tan_y, 1)], dtype=np.float32)
    return np.concatenate((unit * near, unit * far), axis=0)


def box_in_view_space(range_low, range_up, world_view_transform: np.ndarray) -> np.ndarray:
    """grid_utils/utils.py:118-119: row vectors times the transposed world-to-camera matrix."""
    v = np.concatenate((space_box_vertices(range_low, range_up), np.ones((8, 1), dtype=np.float32)), axis=1)
    return np.dot(v, world_view_transform)[:, :3]


def is_overlapping_spacebox_view(range_low, range_up, world_view_transform, fovx, fovy, z_near=0.01, z_far=1e6) -> bool:
    """grid_utils/utils.py:115-137: the origin lies inside (or on) the convex hull of the
    64 pairwise differences exactly when the two bodies share a point."""
    from scipy.spatial import ConvexHull
    box = box_in_view_space(range_low, range_up, world_view_transform)
    fr = frustum_vertices(fovx, fovy, z_near, z_far)
    diff = (box.reshape(8, 1, 3) - fr.reshape(1, 8, 3)).reshape(-1, 3)
    hull = ConvexHull(diff)
    distances = np.dot(hull.equations, np.array((0, 0, 0, 1.0)).reshape(4, 1))
    return bool(np.all(distances <= 0))


# ---------------------------------------------------------------------------------------------
# order of the submodels for one camera: parallel_utils/basic_parallel_trainer/scene_utils.py:220-264
# ---------------------------------------------------------------------------------------------
def relation_vector(camera_center, leaf_paths: Sequence[str], splits: Dict[str, Tuple[int, float]],
                    overlaps: Sequence[bool]) -> np.ndarray:
    """``splits[path] = (split_dim, split position in world units)`` for every inner node;
    ``overlaps[m]`` is the frustum test of leaf m.  The nearer child of every split gets depth 0."""
    c = np.array(camera_center, dtype=np.float64).reshape(-1)[:3]
    node_depth = {"": 0}
    for path, (dim, where) in splits.items():
        right_is_near = c[dim] > where                      # grid_utils/utils.py:279-286
        node_depth[path + "1"] = 0 if right_is_near else 1
        node_depth[path + "0"] = 1 if right_is_near else 0
    listed = []
    for mid, path in enumerate(leaf_paths):
        listed.append((mid, tuple(node_depth[path[:n + 1]] for n in range(len(path)))))
    listed.sort(key=lambda item: item[-1])
    relation = np.zeros(len(leaf_paths), dtype=int) - 1
    for order, (mid, _) in enumerate(listed):
        relation[mid] = order if overlaps[mid] else -1
    if relation.sum() == -len(leaf_paths):                   # scene_utils.py:313-315
        relation[:] = 0
    return relation


# ---------------------------------------------------------------------------------------------
# boundary straddlers: parallel_utils/basic_parallel_trainer/result_aggregator.py:55-121, 263-288
# ---------------------------------------------------------------------------------------------
def straddler_rows(means3D: np.ndarray, scales: np.ndarray, src_low, src_up, dst_low, dst_up) -> np.ndarray:
    """Row numbers (ascending) of the source submodel's Gaussians that are lent to one
    destination: the 3-sigma cube (3 x largest activated scale, floored at 0) reaches one of
    the source box's faces (result_aggregator.py:76-85) and meets the destination box on all
    three axes (:103-106).  All arithmetic in float32, as torch does it."""
    means3D = np.asarray(means3D, dtype=np.float32)
    reach = np.maximum(np.max(np.asarray(scales, dtype=np.float32), axis=-1, keepdims=True) * np.float32(3), np.float32(0))
    max_xyz = means3D + reach
    min_xyz = means3D - reach
    candidate = np.any((max_xyz >= np.asarray(src_up, np.float32)) | (min_xyz <= np.asarray(src_low, np.float32)), axis=-1)
    meets = np.all((max_xyz >= np.asarray(dst_low, np.float32)) & (min_xyz <= np.asarray(dst_up, np.float32)), axis=-1)
    return np.nonzero(candidate & meets)[0]


def merged_rows(own_counts: Sequence[int], lent: Dict[Tuple[int, int], np.ndarray], dst: int) -> List[Tuple[int, np.ndarray]]:
    """The (source submodel, row numbers) blocks that make up destination dst's input, in
    order: its own rows first, then every lender in ascending id (merge_SharedGSInfo,
    result_aggregator.py:263-288, walking a pool filled in ascending source id, :123-141)."""
    blocks = [(dst, np.arange(own_counts[dst], dtype=np.int64))]
    for src in range(len(own_counts)):
        if src != dst:
            blocks.append((src, np.asarray(lent[(src, dst)], dtype=np.int64)))
    return blocks


def merge_fields(fields_by_model: Sequence[Dict[str, np.ndarray]], blocks: List[Tuple[int, np.ndarray]]) -> Dict[str, np.ndarray]:
    """torch.cat of the picked rows, field by field."""
    names = fields_by_model[0].keys()
    return {n: np.concatenate([fields_by_model[src][n][rows] for src, rows in blocks], axis=0) for n in names}


def merge_backward(grad_merged: Dict[str, np.ndarray], blocks: List[Tuple[int, np.ndarray]],
                   shapes_by_model: Sequence[Dict[str, tuple]]) -> List[Dict[str, np.ndarray]]:
    """Adjoint of merge_fields for ONE destination: every block's gradient rows go back to
    the rows they were read from (autograd of indexing followed by cat)."""
    out = [{n: np.zeros(s, dtype=np.float32) for n, s in shapes.items()} for shapes in shapes_by_model]
    at = 0
    for src, rows in blocks:
        for n, g in grad_merged.items():
            out[src][n][rows] += g[at:at + len(rows)]
        at += len(rows)
    return out
