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

import math

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
    # partition_scene_on_device leaves owner and members as tensors on the scene's device


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


def _grid_from_extent(xyz_min: np.ndarray, xyz_max: np.ndarray, scale_max: np.ndarray):
    """low, up, voxel, size of build_grid from the three per-axis extremes (float32, as there)."""
    pad = 3.0 * scale_max.astype(np.float32)
    low = xyz_min.astype(np.float32) - pad
    up = xyz_max.astype(np.float32) + pad
    voxel = (up - low) / np.asarray(SCENE_GRID_SIZE, dtype=low.dtype) - 1e-7
    low, up, voxel = (np.asarray(v, dtype=np.float32) for v in (low, up, voxel))
    size = tuple(max(int((up[i] - low[i]) // voxel[i]), 1) for i in range(3))
    return low, up, voxel, size


def partition_scene_on_device(xyz: torch.Tensor, scales_activated: torch.Tensor, depth: int,
                              rows_per_pass: int = 1 << 24) -> Partition:
    """partition_scene for scenes too large to take through the host (tens to hundreds of millions
    of Gaussians): the per-Gaussian work (voxel histogram, ownership, straddler selection) is done
    with tensor operations on the device the scene lives on, in float32 like the numpy version, and
    gives the same grid, boxes, owners and member lists; the tree itself (a 2048 x 2048 histogram)
    is split on the host.  owner and members come back as tensors on that device."""
    dev = xyz.device
    N = int(xyz.shape[0])
    f32 = lambda t: t.detach().cpu().numpy().astype(np.float32)
    low, up, voxel, size = _grid_from_extent(f32(xyz.min(dim=0).values), f32(xyz.max(dim=0).values),
                                             f32(scales_activated.max(dim=0).values))
    low_t, voxel_t = torch.from_numpy(low).to(dev), torch.from_numpy(voxel).to(dev)
    size_t = torch.tensor(size, device=dev)
    cells = size[0] * size[1] * size[2]
    load = torch.zeros(cells, dtype=torch.int64, device=dev)
    for at in range(0, N, rows_per_pass):
        idx = torch.floor_divide(xyz[at:at + rows_per_pass] - low_t, voxel_t).long()
        ok = ((idx >= 0) & (idx < size_t)).all(dim=1)
        flat = ((idx[:, 0] * size[1] + idx[:, 1]) * size[2] + idx[:, 2])[ok]
        load += torch.bincount(flat, minlength=cells)
    grid = Grid(low, up, voxel, size, load.reshape(size).double().cpu().numpy())
    nodes = build_bvh(grid, depth)
    leaves = sorted((n for n in nodes.values() if n.is_leaf), key=lambda n: n.path)
    K = len(leaves)
    box_low = np.stack([np.asarray(n.low) * grid.voxel.astype(np.float64) + grid.low for n in leaves]).astype(np.float32)
    box_up = np.stack([np.asarray(n.up) * grid.voxel.astype(np.float64) + grid.low for n in leaves]).astype(np.float32)
    lows, ups = torch.from_numpy(box_low).to(dev), torch.from_numpy(box_up).to(dev)

    owner = torch.full((N,), -1, dtype=torch.int64, device=dev)
    for at in range(0, N, rows_per_pass):
        p = xyz[at:at + rows_per_pass]
        part = owner[at:at + rows_per_pass]
        for k in range(K):  # later ids overwrite earlier ones on ties
            part[((p >= lows[k]) & (p <= ups[k])).all(dim=1)] = k
    if bool((owner < 0).any()):
        raise RuntimeError("a Gaussian fell outside every submodel box")

    own = [torch.nonzero(owner == k).squeeze(1) for k in range(K)]
    lent = [[None] * K for _ in range(K)]   # lent[dst][src]
    for src in range(K):
        ids = own[src]
        if ids.numel() == 0:
            continue
        p = xyz[ids]
        r = (3.0 * scales_activated[ids].max(dim=1).values).clamp(min=0.0).unsqueeze(1)
        hi, lo = p + r, p - r
        cand = ((hi >= ups[src]) | (lo <= lows[src])).any(dim=1)
        ids, hi, lo = ids[cand], hi[cand], lo[cand]
        for dst in range(K):
            if dst != src:
                lent[dst][src] = ids[((hi >= lows[dst]) & (lo <= ups[dst])).all(dim=1)]
    members = [torch.cat([own[dst]] + [lent[dst][src] for src in range(K) if src != dst and lent[dst][src] is not None])
               for dst in range(K)]
    return Partition(grid, nodes, leaves, box_low, box_up, owner, members)


_BOX_CORNERS = np.array([[x, y, z] for x in (0, 1) for y in (0, 1) for z in (0, 1)], dtype=np.float32)


def view_frustum_vertices(cam, z_near: Optional[float] = None, z_far: Optional[float] = None) -> np.ndarray:
    """The eight corners, in camera space, of the frustum between z_near and z_far
    (parallel_utils/grid_utils/utils.py:80-112: z_near is at least 0.01, z_far at most 1e6)."""
    near = max(0.01, 0.01 if z_near is None else z_near)
    far = min(1e6, 1e6 if z_far is None else z_far)
    tx, ty = math.tan(cam.FoVx / 2), math.tan(cam.FoVy / 2)
    unit = np.array([(tx, ty, 1), (tx, -ty, 1), (-tx, ty, 1), (-tx, -ty, 1)], dtype=np.float32)
    return np.concatenate((unit * np.float32(near), unit * np.float32(far)), axis=0)


def boxes_overlap_view(low: np.ndarray, up: np.ndarray, cam, z_near: float = 0.01, z_far: float = 1e6) -> np.ndarray:
    """For K world-space boxes (low, up: (K,3)): does the box meet the camera's frustum?

    Same predicate as is_overlapping_SpaceBox_View (parallel_utils/grid_utils/utils.py:115-137),
    which asks whether the origin lies in the convex hull of the Minkowski difference of the two
    vertex sets, i.e. whether the two convex bodies share a point (touching counts).  Decided
    here without a hull: two convex polyhedra are disjoint exactly when one of the face normals
    of either, or one of the cross products of an edge of one with an edge of the other,
    separates their vertex sets.  A box in camera space has 3 face normals and 3 edge directions,
    the frustum 5 face normals and 6 edge directions: 26 candidate axes, all K boxes at once.
    """
    low = np.asarray(low, dtype=np.float32).reshape(-1, 3)
    up = np.asarray(up, dtype=np.float32).reshape(-1, 3)
    corners = np.where(_BOX_CORNERS[None] > 0, up[:, None, :], low[:, None, :])
    w2c_t = cam.world_view_transform.detach().cpu().numpy().astype(np.float32)
    homogeneous = np.concatenate((corners, np.ones(corners.shape[:2] + (1,), dtype=np.float32)), axis=2)
    box = np.dot(homogeneous, w2c_t)[..., :3].astype(np.float64)               # (K,8,3) camera space
    frustum = view_frustum_vertices(cam, z_near, z_far).astype(np.float64)     # (8,3)
    tx, ty = frustum[0, 0] / frustum[0, 2], frustum[0, 1] / frustum[0, 2]

    # edge directions of the box in camera space (images of the world axes)
    box_edges = np.stack((box[:, 4] - box[:, 0], box[:, 2] - box[:, 0], box[:, 1] - box[:, 0]), axis=1)   # (K,3,3)
    box_normals = np.stack((np.cross(box_edges[:, 1], box_edges[:, 2]), np.cross(box_edges[:, 2], box_edges[:, 0]),
                            np.cross(box_edges[:, 0], box_edges[:, 1])), axis=1)
    frustum_normals = np.array([(0, 0, 1), (1, 0, -tx), (-1, 0, -tx), (0, 1, -ty), (0, -1, -ty)], dtype=np.float64)
    frustum_edges = np.array([(1, 0, 0), (0, 1, 0), (tx, ty, 1), (tx, -ty, 1), (-tx, ty, 1), (-tx, -ty, 1)], dtype=np.float64)
    crossed = np.cross(box_edges[:, :, None, :], frustum_edges[None, None, :, :]).reshape(len(box), 18, 3)
    axes = np.concatenate((box_normals, np.broadcast_to(frustum_normals, (len(box), 5, 3)), crossed), axis=1)  # (K,26,3)
    length = np.linalg.norm(axes, axis=2, keepdims=True)
    axes = np.where(length > 1e-12, axes / np.maximum(length, 1e-300), 0.0)    # a vanishing cross product separates nothing

    on_box = np.einsum("kad,kvd->kav", axes, box)
    on_frustum = np.einsum("kad,vd->kav", axes, frustum)
    apart = (on_box.max(axis=2) < on_frustum.min(axis=2)) | (on_frustum.max(axis=2) < on_box.min(axis=2))
    return ~apart.any(axis=1)


def relation_vector(part: Partition, cam, z_near: float = 0.01, z_far: float = 1000.0) -> np.ndarray:
    """Compositing rank of every submodel for this camera, -1 when its box misses the frustum
    between z_near and z_far (defaults: main.py:94-95).  A camera that sees no box at all gets
    rank 0 everywhere (scene_utils.py:313-315)."""
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
    seen = boxes_overlap_view(part.box_low, part.box_up, cam, z_near, z_far)
    for order, (_, mid) in enumerate(keyed):
        if seen[mid]:
            rel[mid] = order
    if (rel < 0).all():
        rel[:] = 0
    return rel


def morton_order(xyz: torch.Tensor, bits: int = 10) -> torch.Tensor:
    """Permutation that lists the points (N,3) along a Z-order curve over their bounding box (`bits` bits per
    axis; ties keep index order).  The reference stores a submodel's Gaussians in the order its loader met them
    (scene/gaussian_nn_module.py:176-192, a boolean mask over the file's order); stored along the curve instead,
    the Gaussians a camera sees lie together in memory, and the per-Gaussian kernels, which read the rows of the
    visible ones only, read runs of rows instead of every third row."""
    if xyz.numel() == 0:
        return torch.zeros(0, dtype=torch.long, device=xyz.device)
    low = xyz.min(dim=0).values
    extent = (xyz.max(dim=0).values - low).clamp_min(1e-12)
    cells = ((xyz - low) / extent * (2 ** bits - 1)).round().to(torch.long).clamp_(0, 2 ** bits - 1)
    code = torch.zeros(xyz.shape[0], dtype=torch.long, device=xyz.device)
    for b in range(bits):
        for axis in range(3):
            code |= ((cells[:, axis] >> b) & 1) << (3 * b + axis)
    return torch.argsort(code, stable=True)

