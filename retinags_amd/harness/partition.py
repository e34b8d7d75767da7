"""Spatial partition of a Gaussian scene into 2**depth axis-aligned submodels, the
sharing of boundary-straddling Gaussians and the per-camera front-to-back order: the
minimum of the reference's scheduler that the one-GPU render -> composite -> backward
loop needs.  Restates, in numpy:
  grid            scene/gaussian_nn_module.py:284-294, parallel_utils/grid_utils/utils.py:154-178
  BVH split       parallel_utils/grid_utils/utils.py:228-263, 334-360 (split axes 0,1,0,1,...; main.py:46-47)
  submodel boxes  parallel_utils/basic_parallel_trainer/trainer4tree_partition.py:174-175
  ownership       scene/gaussian_nn_module.py:176-192
  straddlers      parallel_utils/basic_parallel_trainer/result_aggregator.py:55-121, 263-288
  order vector    parallel_utils/basic_parallel_trainer/scene_utils.py:220-264
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

SCENE_GRID_SIZE = (2048, 2048, 1)
SPLIT_ORDERS = (0, 1)


@dataclass
class Grid:
    low: np.ndarray      # (3,) float32, as broadcast by the reference
    up: np.ndarray
    voxel: np.ndarray
    size: Tuple[int, int, int]
    load: np.ndarray     # (gx, gy, gz) float64 counts


@dataclass
class Node:
    low: Tuple[int, int, int]
    up: Tuple[int, int, int]
    level: int
    path: str
    split_dim: int
    split_position: Optional[int] = None
    children: List["Node"] = field(default_factory=list)

    @property
    def is_leaf(self) -> bool:
        return not self.children


@dataclass
class Partition:
    grid: Grid
    nodes: Dict[str, Node]
    leaves: List[Node]            # sorted by path; index = submodel id
    box_low: np.ndarray           # (K,3) float32 world-space boxes
    box_up: np.ndarray
    owner: np.ndarray             # (N,) submodel id of every Gaussian
    members: List[np.ndarray]     # per submodel: indices into the scene, own Gaussians first,
                                  # then straddlers from other submodels in ascending source id


def build_grid(xyz: np.ndarray, scales_activated: np.ndarray) -> Grid:
    pad = 3.0 * scales_activated.max(axis=0)
    low = xyz.min(axis=0) - pad
    up = xyz.max(axis=0) + pad
    voxel = (up - low) / np.asarray(SCENE_GRID_SIZE, dtype=low.dtype) - 1e-7
    low, up, voxel = (np.asarray(v, dtype=np.float32) for v in (low, up, voxel))
    size = tuple(max(int((up[i] - low[i]) // voxel[i]), 1) for i in range(3))
    load = np.zeros(size, dtype=np.float64)
    idx = ((xyz - low) // voxel).astype(np.int64)
    ok = np.all((idx >= 0) & (idx < np.asarray(size)), axis=1)
    np.add.at(load, tuple(idx[ok].T), 1.0)
    return Grid(low, up, voxel, size, load)


def _split(node: Node, grid: Grid, limit: int) -> List[Node]:
    d = node.split_dim
    if node.up[d] - node.low[d] < 2:
        return []
    sl = tuple(slice(node.low[i], node.up[i]) for i in range(3))
    other = tuple(i for i in range(3) if i != d)
    along = grid.load[sl].sum(axis=other)
    imbalance = np.abs(2.0 * np.cumsum(along) - along.sum())
    s = int(np.argmin(imbalance))
    limit = int(np.clip(limit, 0, len(imbalance) // 2))
    s = int(np.clip(s, limit, len(imbalance) - 1 - limit))
    cut = node.low[d] + s + 1
    node.split_position = cut
    left_up = list(node.up)
    left_up[d] = cut
    right_low = list(node.low)
    right_low[d] = cut
    nd = SPLIT_ORDERS[(node.level + 1) % len(SPLIT_ORDERS)]
    node.children = [Node(node.low, tuple(left_up), node.level + 1, node.path + "0", nd),
                     Node(tuple(right_low), node.up, node.level + 1, node.path + "1", nd)]
    return node.children


def build_bvh(grid: Grid, depth: int) -> Dict[str, Node]:
    root = Node((0, 0, 0), grid.size, 0, "", SPLIT_ORDERS[0])
    queue, nodes = [root], {}
    while queue:
        node = queue.pop(0)
        if node.level < depth:
            queue.extend(_split(node, grid, 2 ** (depth - node.level)))
        nodes[node.path] = node
    return nodes


def _straddler_sources(xyz, radius, low, up):
    """Gaussians of a submodel whose 3-sigma box reaches one of its own faces."""
    return np.any((xyz + radius[:, None] >= up) | (xyz - radius[:, None] <= low), axis=1)


def partition_scene(xyz: torch.Tensor, scales_activated: torch.Tensor, depth: int) -> Partition:
    xyz_np = xyz.detach().cpu().numpy().astype(np.float32)
    sc_np = scales_activated.detach().cpu().numpy().astype(np.float32)
    grid = build_grid(xyz_np, sc_np)
    nodes = build_bvh(grid, depth)
    leaves = sorted((n for n in nodes.values() if n.is_leaf), key=lambda n: n.path)
    K = len(leaves)
    box_low = np.stack([np.asarray(n.low) * grid.voxel.astype(np.float64) + grid.low for n in leaves]).astype(np.float32)
    box_up = np.stack([np.asarray(n.up) * grid.voxel.astype(np.float64) + grid.low for n in leaves]).astype(np.float32)

    owner = np.full(xyz_np.shape[0], -1, dtype=np.int64)
    for k in range(K):  # later ids overwrite earlier ones on ties
        inside = np.all((xyz_np >= box_low[k]) & (xyz_np <= box_up[k]), axis=1)
        owner[inside] = k
    if (owner < 0).any():
        raise RuntimeError("a Gaussian fell outside every submodel box")

    radius = np.clip(3.0 * sc_np.max(axis=1), 0.0, None)
    own = [np.nonzero(owner == k)[0] for k in range(K)]
    members = []
    for dst in range(K):
        parts = [own[dst]]
        for src in range(K):
            if src == dst or own[src].size == 0:
                continue
            ids = own[src]
            p, r = xyz_np[ids], radius[ids]
            cand = _straddler_sources(p, r, box_low[src], box_up[src])
            reach = np.all((p + r[:, None] >= box_low[dst]) & (p - r[:, None] <= box_up[dst]), axis=1)
            parts.append(ids[cand & reach])
        members.append(np.concatenate(parts))
    return Partition(grid, nodes, leaves, box_low, box_up, owner, members)


def _box_may_be_seen(low, up, cam) -> bool:
    """Conservative frustum test: a box is dropped only when all eight corners lie behind
    the near plane or beyond one side plane.  (The reference intersects the exact hulls,
    parallel_utils/grid_utils/utils.py:115-137; a box kept here that it would drop
    renders an empty partial image, which composites as a no-op.)"""
    corners = np.array([[x, y, z, 1.0] for x in (low[0], up[0]) for y in (low[1], up[1]) for z in (low[2], up[2])])
    v = corners @ cam.world_view_transform.cpu().numpy().astype(np.float64)
    z = v[:, 2]
    if np.all(z < 0.01):
        return False
    tx, ty = cam.tanfovx, cam.tanfovy
    for a, t in ((v[:, 0], tx), (v[:, 1], ty)):
        if np.all(a > t * np.maximum(z, 0.0) + 1e-6) and np.all(z > 0):
            return False
        if np.all(a < -t * np.maximum(z, 0.0) - 1e-6) and np.all(z > 0):
            return False
    return True


def relation_vector(part: Partition, cam) -> np.ndarray:
    """Compositing rank of every submodel for this camera, -1 when it cannot be seen."""
    center = cam.camera_center.cpu().numpy().astype(np.float64)
    depth_bit = {"": 0}
    for path, node in part.nodes.items():
        if node.is_leaf or node.split_position is None:
            continue
        d = node.split_dim
        split_world = node.split_position * part.grid.voxel[d] + part.grid.low[d]
        cam_in_right = center[d] > split_world
        depth_bit[path + "1"] = 0 if cam_in_right else 1
        depth_bit[path + "0"] = 1 if cam_in_right else 0
    keyed = []
    for mid, leaf in enumerate(part.leaves):
        keyed.append((tuple(depth_bit[leaf.path[:i + 1]] for i in range(len(leaf.path))), mid))
    keyed.sort(key=lambda t: t[0])
    rel = np.full(len(part.leaves), -1, dtype=np.int64)
    for order, (_, mid) in enumerate(keyed):
        if _box_may_be_seen(part.box_low[mid], part.box_up[mid], cam):
            rel[mid] = order
    if (rel < 0).all():
        rel[:] = 0
    return rel
